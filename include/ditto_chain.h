/*
 * ditto_chain.h — C ABI of the MI355X (gfx950) fused operator-chain library.
 *
 * This is the boundary a Ditto maintainer binds in place of the TVM PackedFunc
 * that `tvm.build(sch, layer.schedule_tensors, "cuda")` returns for a
 * hyper_fusion chain (reference: benchmark/chimera/cuda/bmm_softmax_bmm_cuda.py:26,239,256;
 * src/runtime/graph_runtime.cc:149).  The reference call is
 * `func(*inputs, *outputs)` with destination passing: the caller owns every
 * buffer and the callee allocates nothing the caller can see.  The same holds
 * here: all data pointers are DEVICE pointers owned by the caller; the library
 * enqueues one kernel on the given HIP stream and returns without
 * synchronising.  Nothing is thrown across this boundary: every entry point
 * returns 0 on success or a negative DITTO_E* code, and ditto_last_error()
 * returns the calling thread's last message.
 *
 * Plain C: no HIP or torch types appear in the signatures (a stream is passed
 * as void*, i.e. a hipStream_t; NULL is the default stream).
 */
#ifndef DITTO_CHAIN_H_
#define DITTO_CHAIN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: ditto_conv_chain_desc gained tile_variant (the kernel to force; run-time switches in the environment are gone) */
#define DITTO_CHAIN_ABI_VERSION 2

/* error codes */
#define DITTO_OK 0
#define DITTO_EINVAL (-1)      /* descriptor / shape / alignment not valid          */
#define DITTO_EUNSUPPORTED (-2)/* valid chain, but no kernel for this dtype / shape */
#define DITTO_EHIP (-3)        /* a HIP runtime call failed                         */
#define DITTO_EWORKSPACE (-4)  /* workspace too small                               */

/* element types (reference: the in_dtype / acc_dtype strings of the chain
 * builders, benchmark/chimera/cuda/bmm_bmm_cuda.py:273-288) */
typedef enum ditto_dtype {
  DITTO_F16 = 0,
  DITTO_BF16 = 1,
  DITTO_F32 = 2,
  DITTO_I8 = 3,
  DITTO_I32 = 4,
  DITTO_F64 = 5
} ditto_dtype;

/* The op on the single path between the two contractions
 * (reference: TensorizeHyperFusionState::inter_path, src/auto_tensorize/hyper_fusion.cc:51-216). */
typedef enum ditto_inter_op {
  DITTO_INTER_CAST = 0,    /* mid = cast_in(acc)                      bmm_bmm_cuda.py:114-118 (int8: the
                              accumulator's low byte, what astype("int8") keeps)                    */
  DITTO_INTER_RELU = 1,    /* mid = cast_in(max(acc,0))               conv_relu_conv_relu_fuse_hw_cuda.py:134-142 */
  DITTO_INTER_SOFTMAX = 2, /* mid = softmax(scale*acc) over L, online  bmm_chain.py:63-103 (exp + ones column + divide) */
  DITTO_INTER_REQUANT = 3  /* mid = sat_i8(rne(acc * scale[col]))      int8 chain; not in the reference,
                              whose int8 chain wraps with astype("int8") (bmm_bmm_cuda.py:116)   */
} ditto_inter_op;

/* How the second operand of the first contraction is laid out in memory. */
typedef enum ditto_b_layout {
  DITTO_B_KL = 0, /* B[batch][K][L], L contiguous: the reference's placeholder layout
                     (bmm_bmm_cuda.py:87, bmm_chain.py:29-31 `key[batch,K,L]`)          */
  DITTO_B_LK = 1  /* B stored as [batch][L][K], K contiguous: a transposed view of the
                     above (what self_attention.py:55-57 transposes FROM); no copy made */
} ditto_b_layout;

/*
 * Batched two-contraction chain  F[b] = epilogue( inter( A[b]·B[b] ) · C[b] ).
 * Names follow the reference builders: A[batch,M,K], B[batch,K,L], C[batch,L,N],
 * F[batch,M,N] (bmm_bmm_cuda.py:69-149, bmm_chain.py:5-105).
 * Strides are in ELEMENTS.  Rows must be contiguous (innermost stride 1).
 */
typedef struct ditto_bmm_chain_desc {
  int32_t abi_version;   /* DITTO_CHAIN_ABI_VERSION */
  int32_t in_dtype;      /* ditto_dtype of A, B, C                                    */
  int32_t acc_dtype;     /* DITTO_F32 (fp16 / bf16 / fp32 chains; DITTO_F16 with fp16 operands is
                            accepted and served in fp32), DITTO_F64 (fp64), DITTO_I32 (int8) */
  int32_t out_dtype;     /* in_dtype (reference: F cast to in_dtype) or acc_dtype      */
  int32_t inter_op;      /* ditto_inter_op                                            */
  int32_t b_layout;      /* ditto_b_layout                                            */
  int64_t batch, M, N, K, L;
  int64_t a_batch_stride, a_row_stride; /* A[b][m][k] = a + b*abs + m*ars + k          */
  int64_t b_batch_stride, b_row_stride; /* KL: B[b][k][l] = b + b*bbs + k*brs + l
                                           LK: B[b][k][l] = b + b*bbs + l*brs + k      */
  int64_t c_batch_stride, c_row_stride; /* C[b][l][n]                                  */
  int64_t f_batch_stride, f_row_stride; /* F[b][m][n]                                  */
  float softmax_scale;   /* DITTO_INTER_SOFTMAX only; the reference uses 1.0           */
  float requant_scale;   /* DITTO_INTER_REQUANT: scale of every column when `aux` is NULL */
  int32_t tile_variant;  /* 0: the library's per-shape table picks the kernel variant; else a
                            `ditto_tile_param.variant` id to force (the counterpart of passing
                            an explicit CUDATensorizeParam, hyper_fusion.cc:586-607);
                            DITTO_EINVAL if that variant cannot run the shape              */
  int32_t relu_out;      /* 1: ReLU on the second accumulator before the final cast (an activation layer
                            fused into the chain, python/ditto/chimera/graph_fusion.py:4-52); cast / relu
                            chains on fp16, bf16, fp32; else 0 */
  /* Two-level batch (fp16/bf16 chains): batch entry z = zo * batch_inner + zi lives at
   * zo * x_batch_stride_outer + zi * x_batch_stride.  This is how an attention caller hands
   * over [batch, heads] without the reshape/transpose copies of
   * nn/module/self_attention.py:47-57,71-73: heads are the inner level with stride head_dim,
   * the outer stride is one sequence of the packed projection.  batch_inner = 0 (or = batch):
   * single level, the outer strides are ignored. */
  int64_t batch_inner;
  int64_t a_batch_stride_outer, b_batch_stride_outer, c_batch_stride_outer, f_batch_stride_outer;
} ditto_bmm_chain_desc;

/*
 * conv -> conv chain on plain NCHW tensors (reference forms:
 * testing/hyper_fusion/conv_relu_conv_relu_fuse_hw_cuda.py:17-262 for NCHW,
 * benchmark/chimera/cuda/conv3x3_conv1x1_cuda.py:77-172 for the chain; shape
 * tuple as python_test/auto_tensorize/test_hyper_fusion.py:51-192).
 *   X[N][C0][H][W], W1[C1][C0 / groups1][R1][S1], W2[C2][C1][R2][S2] -> Y[N][C2][P2][Q2]
 */
typedef struct ditto_conv_chain_desc {
  int32_t abi_version;
  int32_t in_dtype, acc_dtype, out_dtype;
  int32_t inter_op;      /* DITTO_INTER_CAST or DITTO_INTER_RELU */
  int32_t relu_out;      /* 1: ReLU after the second convolution too */
  int64_t N, C0, H, W;
  int64_t C1, R1, S1, pad1, stride1;
  int64_t C2, R2, S2, pad2, stride2;
  int64_t groups1;       /* groups of the first convolution: 1 (or 0) dense; C0: depthwise with
                            C1 / C0 outputs per input channel, W1[C1][1][R1][S1]
                            (benchmark/chimera/cuda/depthwise3x3_conv1x1_small_channel_cuda.py:77-169,
                            `factor` = C1 / C0); then R1 * S1 <= 9, the second convolution is 1x1
                            and C1 / C0 is 1, 2, 4 or a multiple of 8 */
  int32_t tile_variant;  /* 0: the library's per-shape rules pick the kernel; else the kernel to force, the
                            counterpart of an explicit CUDATensorizeParam (hyper_fusion.cc:586-607): either a
                            `ditto_tile_param.variant` id as ditto_conv_chain_select_tile reported it, or a
                            family id (a multiple of 100) that leaves the tile inside the family to the library:
                              3000 general kernel, 1x1 second convolution (31xx: 16-channel chunks)
                              3500 general kernel, second convolution up to 3x3 through LDS
                              3600 conv1x1 -> conv3x3, persistent workgroups, W2 resident in LDS
                              3700 conv3x3 -> conv1x1 row pipeline        3800 conv1x1 -> conv3x3 row pipeline
                              4000 depthwise -> conv1x1, tile kernels (40xx = 4000 + 10 * output tiles + mode)
                              4024 / 4025 depthwise row-streaming kernels (multiplier 1 / 16)
                            DITTO_EINVAL if that kernel cannot run the chain; with a forced kernel a call
                            whose pointers or workspace the kernel cannot take fails instead of falling
                            back to the general kernel */
  int32_t reserved0;     /* 0 */
} ditto_conv_chain_desc;

/* Tile choice reported back to the host; the static per-shape table replaces
 * CUDATensorizeParam and its search (hyper_fusion.cc:586-607,
 * chimera_integrate.py:298-449). */
typedef struct ditto_tile_param {
  int32_t block_threads;  /* threads per workgroup (multiple of 64)              */
  int32_t block_m;        /* rows of the chain output one workgroup owns         */
  int32_t block_l;        /* extent of the intermediate processed per step       */
  int32_t block_n;        /* columns of the chain output one workgroup owns      */
  int32_t head_pad;       /* K and N padded to this inside the kernel (0: n/a)   */
  int32_t lds_bytes;      /* dynamic LDS per workgroup                           */
  int32_t grid_x, grid_y, grid_z;
  int32_t variant;        /* kernel variant id: fp16/bf16 chains head_pad*10 + q, with
                             q = 1|2: four waves owning 32*q rows each; eight waves owning
                             32 rows each: q = 8 (phases staggered between the two waves of a
                             SIMD), q = 9 (software pipelined), q = 6 (16x16x32 MFMA), q = 7 (the same kernel with 384-row workgroups, 48 rows
                             per wave, for the first row blocks of a batch entry and 256-row ones
                             for the rest; block_m reports 384); four waves on the 16x16x32 MFMA
                             with 64-row workgroups (head_pad 64, either layout of B): q = 4 (a
                             wave owns 16 rows and all keys), q = 5 (32 rows and half the keys of
                             every tile); conv chains: the ids listed at
                             ditto_conv_chain_desc.tile_variant; fp32 / fp64 1000 / 1001; int8
                             8000 + 10 * (row tiles of 32) + ring depth */
} ditto_tile_param;

/* ---- entry points ------------------------------------------------------- */

/* Library / ABI version (DITTO_CHAIN_ABI_VERSION of the build). */
int ditto_chain_abi_version(void);

/* Last error message of the calling thread ("" if none). */
const char* ditto_last_error(void);

/* Tile the library would use for this chain; also validates the descriptor.
 * Replaces the parameter choice of chimera_integrate.py:452-478.  Rules that weigh workgroups against
 * compute units use the current device's count, as the run calls do (256 where the process has no
 * device), so the answer is the kernel a run on this device takes. */
int ditto_bmm_chain_select_tile(const ditto_bmm_chain_desc* desc, ditto_tile_param* out);
int ditto_conv_chain_select_tile(const ditto_conv_chain_desc* desc, ditto_tile_param* out);

/* Bytes of device workspace the run call can use.  BMM chains: 0 (the reference's
 * generated code allocates an fp32 E_frag[B,M,ext_N] internally,
 * evaluation/asplos/ncu_summary_chimera_bmm_softmax_bmm.txt:8).  conv chain: room for
 * the first convolution's weights repacked in channel blocks -- the reference's
 * placeholders are already packed that way by the host
 * (conv3x3_conv1x1_cuda.py:99-103); 0 if the descriptor is invalid. */
size_t ditto_bmm_chain_workspace_bytes(const ditto_bmm_chain_desc* desc);
size_t ditto_conv_chain_workspace_bytes(const ditto_conv_chain_desc* desc);

/*
 * Run one fused chain: replaces `func(A, B, C, F)` of the built PackedFunc
 * (bmm_bmm_cuda.py:256, bmm_softmax_bmm_cuda.py:256).
 *   a, b, c : inputs (device), read-only
 *   aux     : DITTO_INTER_REQUANT: fp32 scale[L], one per intermediate column:
 *             mid = saturate_to_[-128,127](round_to_nearest_even((float)acc * scale[l]));
 *             NULL to use desc->requant_scale for every column.  Other chains: NULL
 *   f       : output (device), must not alias an input
 * in_dtype DITTO_F16 / DITTO_BF16: the MFMA chains (cast, relu, softmax);
 * DITTO_F32 / DITTO_F64 (the ("80", "float64", "float64") row): the reference's fp32 configurations
 * (python_test/auto_tensorize/test_hyper_fusion.py:16-21; the fp32 BMM -> softmax -> BMM of
 * benchmark/chimera/cpu/bmm_softmax_bmm.py:64-170), cast / relu / softmax, K, N <= 128;
 * DITTO_I8: the requantised chain.
 */
int ditto_bmm_chain_run(const ditto_bmm_chain_desc* desc, const void* a, const void* b,
                        const void* c, const void* aux, void* f, void* workspace,
                        size_t workspace_bytes, void* stream);

/* Run one fused conv->conv chain: replaces `func(Img, W1, W2, Out)`
 * (conv3x3_conv1x1_cuda.py:296-305).
 *   workspace : NULL, or ditto_conv_chain_workspace_bytes() bytes of device memory,
 *               16-byte aligned.  Given, a small kernel repacks w1 into it ahead of the
 *               fused kernel on `stream` (every call; calls that share a workspace must
 *               not overlap).  NULL: the fused kernel re-lays w1 out itself, slower.
 *               DITTO_EWORKSPACE if non-NULL and too small. */
int ditto_conv_chain_run(const ditto_conv_chain_desc* desc, const void* x, const void* w1,
                         const void* w2, void* y, void* workspace, size_t workspace_bytes,
                         void* stream);

/* The same call in two steps, for weights that stay fixed over many calls (inference): the
 * reference's drivers are handed weights the host has already packed
 * (conv3x3_conv1x1_cuda.py:99-103, :289-292), outside the timed function.
 *   ditto_conv_chain_prepare      : only the weight repacking kernel, into `workspace`
 *                                   (a no-op for depthwise chains, which use no workspace);
 *   ditto_conv_chain_run_prepared : only the fused kernel, reading the workspace a prepare call
 *                                   (same descriptor, same w1 / w2) has filled; the workspace is
 *                                   read-only here, so such calls may overlap.  w1 / w2 must still
 *                                   be passed (a 1x1 second convolution reads w2 directly, a
 *                                   1x1 first convolution in front of a 3x3 one w1).
 * DITTO_EWORKSPACE if the chain takes a workspace and none (or too small a one) is given. */
int ditto_conv_chain_prepare(const ditto_conv_chain_desc* desc, const void* w1, const void* w2,
                             void* workspace, size_t workspace_bytes, void* stream);
int ditto_conv_chain_run_prepared(const ditto_conv_chain_desc* desc, const void* x, const void* w1,
                                  const void* w2, void* y, void* workspace, size_t workspace_bytes,
                                  void* stream);

/*
 * ditto_conv_chain_run for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the
 * reference.  Same kernels and results as ditto_conv_chain_run with a workspace, but the
 * repacked weights go into a device array inside the library (DITTO_STATIC_WORKSPACE_BYTES per
 * GPU, held until the process ends) and the call allocates nothing.
 *   - DITTO_EWORKSPACE if ditto_conv_chain_workspace_bytes(desc) exceeds that size;
 *   - every call on one GPU shares that GPU's array: calls that overlap on one GPU (two streams,
 *     two threads) race; calls on one stream are ordered and safe;
 *   - the array keeps the last call's contents; each call rewrites all it reads;
 *   - the first call on a device takes the array's address and sets the kernels' LDS limits (host-side
 *     set-up): make it outside any stream capture.  Later calls only launch kernels and can be captured.
 */
#define DITTO_STATIC_WORKSPACE_BYTES (4u << 20)
int ditto_conv_chain_run_static(const ditto_conv_chain_desc* desc, const void* x, const void* w1,
                                const void* w2, void* y, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DITTO_CHAIN_H_ */
