// Instantiates the conv chain kernels for one element type.
// Compiled with -DDITTO_INST_T=<f16|bf16> -DDITTO_INST_NAME=<symbol> -DDITTO_PACK_NAME=<symbol>.
#include "conv_chain.h"

namespace ditto {

// c1_tiles in {1, 2, 4, 8} (32 intermediate channels each), ch in {32, 16} input channels per chunk
hipError_t DITTO_INST_NAME(int c1_tiles, int ch, const ConvChainArgs& args, hipStream_t stream) {
  typedef DITTO_INST_T T;
#define DITTO_CASE(C1T, PXW)                                                         \
  if (c1_tiles == C1T)                                                               \
    return ch == 32 ? launch_conv_chain<T, C1T, PXW, 32>(args, stream) : launch_conv_chain<T, C1T, PXW, 16>(args, stream);
  DITTO_CASE(1, 2)
  DITTO_CASE(2, 2)
  DITTO_CASE(4, 2)
  DITTO_CASE(8, 1)
#undef DITTO_CASE
  return hipErrorInvalidValue;
}

hipError_t DITTO_PACK_NAME(int c1_tiles, int ch, const ConvChainArgs& args, void* out, hipStream_t stream) {
  return launch_pack_conv_w1<DITTO_INST_T>(args, 32 * c1_tiles, ch, out, stream);
}

}  // namespace ditto
