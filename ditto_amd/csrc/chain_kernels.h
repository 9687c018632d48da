// Launchers defined in the per-variant translation units.
#pragma once
#include <hip/hip_runtime.h>

#include "bmm_chain_fp.h"
#include "conv_chain.h"
#include "conv_chain_resident.h"
#include "conv_rows.h"
#include "dw_conv_chain.h"
#include "dw_rows.h"
#include "dw16_rows.h"
#include "gemm_chain_f32.h"
#include "gemm_chain_i8.h"

namespace ditto {

// bmm_chain_fp_inst.hip, one object per (element type, inter-op)
hipError_t launch_f16_cast(int d_pad, int q, bool b_kl, const BmmChainArgs& args, hipStream_t stream);
hipError_t launch_f16_softmax(int d_pad, int q, bool b_kl, const BmmChainArgs& args, hipStream_t stream);
hipError_t launch_bf16_cast(int d_pad, int q, bool b_kl, const BmmChainArgs& args, hipStream_t stream);
hipError_t launch_bf16_softmax(int d_pad, int q, bool b_kl, const BmmChainArgs& args, hipStream_t stream);

// conv_chain_inst.hip, one object per element type; c1_tiles in {1, 2, 4, 8}
// ch in {32, 16}: input channels per staged chunk
hipError_t launch_conv_f16(int c1_tiles, int ch, const ConvChainArgs& args, hipStream_t stream);
hipError_t launch_conv_bf16(int c1_tiles, int ch, const ConvChainArgs& args, hipStream_t stream);
// W1 -> the chunked layout the chain kernel loads directly (conv_w1_chunk_bytes per chunk)
hipError_t pack_conv_w1_f16(int c1_tiles, int ch, const ConvChainArgs& args, void* out, hipStream_t stream);
hipError_t pack_conv_w1_bf16(int c1_tiles, int ch, const ConvChainArgs& args, void* out, hipStream_t stream);
// second convolution larger than 1x1 (32-channel chunks; c1_tiles in {1, 2, 4}; px2 in {1, 2})
hipError_t launch_conv2_f16(int c1_tiles, int px2, const ConvChainArgs& args, hipStream_t stream);
hipError_t launch_conv2_bf16(int c1_tiles, int px2, const ConvChainArgs& args, hipStream_t stream);
hipError_t pack_conv_w2_f16(int c1_tiles, const ConvChainArgs& args, void* out1, void* out2, hipStream_t stream);
hipError_t pack_conv_w2_bf16(int c1_tiles, const ConvChainArgs& args, void* out1, void* out2, hipStream_t stream);
// 1x1 -> 3x3 with at most 64 channels: persistent kernel, W2 resident in LDS (conv_chain_resident.h)
hipError_t launch_conv_resident_f16(const ConvResidentArgs& args, int grid, hipStream_t stream);
hipError_t launch_conv_resident_bf16(const ConvResidentArgs& args, int grid, hipStream_t stream);
hipError_t pack_conv_w2_resident_f16(const void* w2, void* out, int C1, int C2, hipStream_t stream);
hipError_t pack_conv_w2_resident_bf16(const void* w2, void* out, int C1, int C2, hipStream_t stream);
// 3x3 -> 1x1 with at most 64 -> 64 -> 256 channels, rows of at most 64 pixels: the row pipeline (conv_rows.h)
hipError_t launch_conv_rows_f16(const ConvRowsArgs& args, hipStream_t stream);
hipError_t launch_conv_rows_bf16(const ConvRowsArgs& args, hipStream_t stream);
// depthwise first convolution (dw_conv_chain.h); c2_tiles in {1, 2, 4, 8}; mode 0 | 1: plain kernel,
// vector-ALU depthwise stage (1: multiplier a multiple of 8); 2: persistent kernel, MFMA depthwise
// stage (multiplier a multiple of 16); 3: persistent kernel, vector-ALU stage (3x3, multiplier 1, 2, 4, 8)
hipError_t launch_dw_conv_f16(int c2_tiles, int mode, const DwConvArgs& args, hipStream_t stream);
hipError_t launch_dw_conv_bf16(int c2_tiles, int mode, const DwConvArgs& args, hipStream_t stream);
// depthwise 3x3 (multiplier 1) -> 1x1, at most 32 -> 64 channels, rows of at most 128 pixels (dw_rows.h)
hipError_t launch_dw_rows_f16(const DwRowsArgs& args, hipStream_t stream);
hipError_t launch_dw_rows_bf16(const DwRowsArgs& args, hipStream_t stream);
// depthwise 3x3 (multiplier 16) -> 1x1, at most 32 -> 512 -> 64 channels, rows of at most 120 pixels (dw16_rows.h)
hipError_t launch_dw16_rows_f16(const Dw16RowsArgs& args, hipStream_t stream);
hipError_t launch_dw16_rows_bf16(const Dw16RowsArgs& args, hipStream_t stream);

}  // namespace ditto
