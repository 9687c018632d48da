// Instantiates the conv chain kernels for one element type.
// Compiled with -DDITTO_INST_T=<f16|bf16> and -DDITTO_{INST,PACK,INST2,PACK2,RES,PACKRES,DW}_NAME=<symbol>.
#include "conv_chain.h"
#include "conv_chain_resident.h"
#include "dw_conv_chain.h"

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

// second convolution larger than 1x1: c1_tiles in {1, 2, 4, 8}, px2 in {1, 2} output-pixel tiles per wave (eight
// tiles of intermediate channels leave 128 pixel slots: one output-pixel tile per wave)
hipError_t DITTO_INST2_NAME(int c1_tiles, int px2, const ConvChainArgs& args, hipStream_t stream) {
  typedef DITTO_INST_T T;
  if (c1_tiles == 1) return px2 == 1 ? launch_conv_chain<T, 1, 2, 32, 1>(args, stream) : launch_conv_chain<T, 1, 2, 32, 2>(args, stream);
  if (c1_tiles == 2) return px2 == 1 ? launch_conv_chain<T, 2, 2, 32, 1>(args, stream) : launch_conv_chain<T, 2, 2, 32, 2>(args, stream);
  if (c1_tiles == 4) return px2 == 1 ? launch_conv_chain<T, 4, 2, 32, 1>(args, stream) : launch_conv_chain<T, 4, 2, 32, 2>(args, stream);
  if (c1_tiles == 8 && px2 == 1) return launch_conv_chain<T, 8, 1, 32, 1>(args, stream);
  return hipErrorInvalidValue;
}

hipError_t DITTO_PACK2_NAME(int c1_tiles, const ConvChainArgs& args, void* out1, void* out2, hipStream_t stream) {
  return launch_pack_conv_w12<DITTO_INST_T>(args, 32 * c1_tiles, 32, out1, out2, stream);
}

// 1x1 first, 3x3 second convolution, at most 64 channels: persistent kernel with W2 resident in LDS
hipError_t DITTO_RES_NAME(const ConvResidentArgs& args, int grid, hipStream_t stream) {
  return launch_conv_chain_resident<DITTO_INST_T>(args, grid, stream);
}
hipError_t DITTO_PACKRES_NAME(const void* w2, void* out, int C1, int C2, hipStream_t stream) {
  return pack_conv_w2_resident<DITTO_INST_T>(w2, out, C1, C2, stream);
}

// depthwise first convolution: c2_tiles in {1, 2, 4, 8} (32 output channels each); mode 0 | 1: plain
// kernel with a vector-ALU depthwise stage (1: the multiplier is a multiple of 8); 2 | 3: persistent
// kernel with the depthwise stage on the matrix cores (2) or the vector ALU (3)
hipError_t DITTO_DW_NAME(int c2_tiles, int mode, const DwConvArgs& args, hipStream_t stream) {
  typedef DITTO_INST_T T;
#define DITTO_CASE(C2T, PXW)                                                                    \
  if (c2_tiles == C2T) {                                                                        \
    if (mode >= 2)                                                                              \
      return launch_dw_conv_mfma<T, C2T, dw_mfma_pxw(C2T), dw_mfma_groups(C2T)>(args, args.grid, mode == 3, stream); \
    return mode == 1 ? launch_dw_conv_chain<T, C2T, PXW, true>(args, stream)                    \
                     : launch_dw_conv_chain<T, C2T, PXW, false>(args, stream);                  \
  }
  DITTO_CASE(1, 2)
  DITTO_CASE(2, 2)
  DITTO_CASE(4, 2)
  DITTO_CASE(8, 1)
#undef DITTO_CASE
  return hipErrorInvalidValue;
}

}  // namespace ditto
