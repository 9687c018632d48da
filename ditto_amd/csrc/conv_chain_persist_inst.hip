// Instantiates the persistent conv chain kernel for one element type.
// Compiled with -DDITTO_INST_T=<f16|bf16> and -DDITTO_PERSIST_NAME=<symbol>.
#include "conv_chain_persist.h"

namespace ditto {

// c1_tiles in {1, 2}, ch in {32, 64} (all input channels, padded); 256 output channels (padded);
// square first filters of 1 or 3 taps a side (args.R == args.S).  (Four output-channel tiles or 5x5
// filters made the compiler spill the unrolled first convolution to scratch: not instantiated.)
hipError_t DITTO_PERSIST_NAME(int c1_tiles, int ch, int c2_tiles, const ConvChainArgs& args, int grid, hipStream_t stream) {
  typedef DITTO_INST_T T;
  if (args.R != args.S || c2_tiles != 8) return hipErrorInvalidValue;
#define DITTO_CASE(C1T, CH)                                                                   \
  if (c1_tiles == C1T && ch == CH) {                                                          \
    if (args.R == 1) return launch_conv_chain_persist<T, C1T, CH, 8, 1>(args, grid, stream);  \
    if (args.R == 3) return launch_conv_chain_persist<T, C1T, CH, 8, 3>(args, grid, stream);  \
    return hipErrorInvalidValue;                                                              \
  }
  DITTO_CASE(1, 32)
  DITTO_CASE(1, 64)
  DITTO_CASE(2, 32)
  DITTO_CASE(2, 64)
#undef DITTO_CASE
  return hipErrorInvalidValue;
}

}  // namespace ditto
