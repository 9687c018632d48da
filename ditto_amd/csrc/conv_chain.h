// Fused conv(RxS) -> cast|relu -> conv(1x1) chain on NCHW tensors, fp16 / bf16, gfx950.
//
// Reference chain: benchmark/chimera/cuda/conv3x3_conv1x1_cuda.py:77-172 (conv -> cast ->
// conv, fp32 accumulate), ReLU variant conv_relu_conv_relu_fuse_hw_cuda.py:134-142 (ReLU on
// the accumulator, then cast).  The reference takes pre-padded images and weights packed
// in 16-channel blocks; here the plain NCHW / KCRS tensors are consumed directly and
// re-laid out while they are staged into LDS.
//
// Both convolutions are computed TRANSPOSED as implicit GEMMs whose MFMA column index is
// the output pixel:
//     mid^T[c1][pix] = sum_{r,s,c0} W1[c1][c0][r][s] * X[c0][pix shifted by (r,s)]
//     out^T[c2][pix] = sum_{c1}     W2[c2][c1]       * cast(mid^T[c1][pix])
// so the accumulator registers of the first (lane = pixel, 16 channels per 32x32 tile) are,
// after the cast, exactly the B operand of the second: the intermediate feature map never
// leaves VGPRs, and a lane's results for one output channel are consecutive pixels, i.e.
// contiguous in NCHW.
//
// A workgroup (4 waves) owns TH output rows x TW output columns of one image
// (TH*TW <= 128*PXW pixel slots, 32*PXW per wave) and all C1 / C2 channels.  Input channels
// are walked in chunks of 16: the halo tile X[16][rows_in][cols_in] is staged to LDS as
// [row][col][channel] and the weight chunk as [r*S+s][c1][channel], so that both MFMA
// operands are 16-byte LDS reads.  W2 is read straight from global memory (it is small and
// shared by every workgroup, so it stays in L2/L1).
#pragma once
#include "common.h"

namespace ditto {

struct ConvChainArgs {
  const void* x;
  const void* w1;
  const void* w2;
  void* y;
  int N, C0, H, W;
  int C1, R, S, pad, stride;
  int C2;
  int P, Q;          // output extent of both convolutions (conv2 is 1x1, stride 1)
  int TH, TW;        // output tile per workgroup
  int tiles_h, tiles_w;
  int rows_in, cols_in;  // halo tile extent
  int relu_mid, relu_out, out_f32;
};

constexpr int kConvCh = 16;       // input channels per chunk = one MFMA k step
constexpr int kConvChStr = 24;    // LDS stride of a channel vector: 16 + 8 pad (48 B, conflict-free)

__host__ __device__ inline int conv_chain_lds_bytes(int rows_in, int cols_in, int RS, int C1p) {
  return (rows_in * cols_in + RS * C1p) * kConvChStr * 2;
}

template <typename T, int C1T, int PXW>
__global__ __launch_bounds__(256) void conv_chain_kernel(ConvChainArgs p) {
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  constexpr int C1p = 32 * C1T;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* const Xs = reinterpret_cast<T*>(smem_raw);                       // [rows_in][cols_in][24]
  T* const Ws = Xs + p.rows_in * p.cols_in * kConvChStr;              // [R*S][C1p][24]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, g = lane >> 5;
  const int RS = p.R * p.S;

  // workgroup -> (image, tile row, tile column); neighbouring ids share an image
  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
  const int tiles = p.tiles_h * p.tiles_w;
  const int n = lid / tiles;
  const int th = (lid % tiles) / p.tiles_w, tw = (lid % tiles) % p.tiles_w;
  const int p0 = th * p.TH, q0 = tw * p.TW;
  const int h0 = p0 * p.stride - p.pad, w0 = q0 * p.stride - p.pad;  // input coords of the halo origin

  const T* __restrict__ Xg = reinterpret_cast<const T*>(p.x) + (long long)n * p.C0 * p.H * p.W;
  const T* __restrict__ W1g = reinterpret_cast<const T*>(p.w1);
  const T* __restrict__ W2g = reinterpret_cast<const T*>(p.w2);

  // pixel slots of this lane: slot = 32*(PXW*wave + j) + ln  ->  (ph, pw) inside the tile
  int xoff[PXW];   // LDS element offset of the lane's pixel at (r,s) = (0,0)
  bool valid[PXW];
  int opix[PXW];   // offset of the pixel inside one output channel plane
#pragma unroll
  for (int j = 0; j < PXW; ++j) {
    const int slot = 32 * (PXW * wave + j) + ln;
    const int ph = slot / p.TW, pw = slot % p.TW;
    valid[j] = ph < p.TH && (p0 + ph) < p.P && (q0 + pw) < p.Q;
    const int phc = valid[j] ? ph : 0, pwc = valid[j] ? pw : 0;
    xoff[j] = ((phc * p.stride) * p.cols_in + pwc * p.stride) * kConvChStr + 8 * g;
    opix[j] = (p0 + phc) * p.Q + q0 + pwc;
  }

  f32x16 acc[C1T][PXW];
#pragma unroll
  for (int c = 0; c < C1T; ++c)
#pragma unroll
    for (int j = 0; j < PXW; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[c][j][r] = 0.f;

  const int xelems = kConvCh * p.rows_in * p.cols_in;
  const int welems = C1p * kConvCh * RS;
  const T zero = (T)0.f;

  for (int c0 = 0; c0 < p.C0; c0 += kConvCh) {
    __syncthreads();  // everyone is done reading the previous chunk
    // ---- stage X[c0..c0+15][halo] as [row][col][channel]; consecutive threads read along w
    for (int e = tid; e < xelems; e += 256) {
      const int c = e / (p.rows_in * p.cols_in);
      const int rem = e - c * (p.rows_in * p.cols_in);
      const int ri = rem / p.cols_in, ci = rem - ri * p.cols_in;
      const int h = h0 + ri, w = w0 + ci;
      T v = zero;
      if (c0 + c < p.C0 && h >= 0 && h < p.H && w >= 0 && w < p.W)
        v = Xg[((long long)(c0 + c) * p.H + h) * p.W + w];
      Xs[(ri * p.cols_in + ci) * kConvChStr + c] = v;
    }
    // ---- stage W1[c1][c0..c0+15][r][s] as [r*S+s][c1][channel]; for one c1 the 16*RS
    //      source elements are contiguous
    for (int e = tid; e < welems; e += 256) {
      const int c1 = e / (kConvCh * RS);
      const int rem = e - c1 * (kConvCh * RS);
      const int c = rem / RS, rs = rem - c * RS;
      T v = zero;
      if (c1 < p.C1 && c0 + c < p.C0) v = W1g[((long long)c1 * p.C0 + c0 + c) * RS + rs];
      Ws[(rs * C1p + c1) * kConvChStr + c] = v;
    }
    __syncthreads();
    // ---- first convolution: one MFMA k step (16 channels) per filter tap
    for (int r = 0; r < p.R; ++r)
      for (int s = 0; s < p.S; ++s) {
        const int tap = (r * p.cols_in + s) * kConvChStr;
        V8 xf[PXW];
#pragma unroll
        for (int j = 0; j < PXW; ++j) xf[j] = *reinterpret_cast<const V8*>(Xs + xoff[j] + tap);
        const T* wrow = Ws + ((r * p.S + s) * C1p + ln) * kConvChStr + 8 * g;
#pragma unroll
        for (int c = 0; c < C1T; ++c) {
          const V8 wf = *reinterpret_cast<const V8*>(wrow + 32 * c * kConvChStr);
#pragma unroll
          for (int j = 0; j < PXW; ++j) acc[c][j] = Elem<T>::mfma32(wf, xf[j], acc[c][j]);
        }
      }
  }

  // ---- inter op on the accumulators, cast: mid^T tile (c, j) regs 8(u%2)..+7 are the
  // B operand of k step u (channels 16u + 4g + {0..3} and 16u + 8 + 4g + {0..3})
  V8 pf[2 * C1T][PXW];
#pragma unroll
  for (int c = 0; c < C1T; ++c)
#pragma unroll
    for (int j = 0; j < PXW; ++j)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[e] = acc[c][j][8 * hh + e];
          if (p.relu_mid) v[e] = fmaxf(v[e], 0.f);
        }
        typename Elem<T>::v2 a0 = cvt2<T>(v[0], v[1]), a1 = cvt2<T>(v[2], v[3]);
        typename Elem<T>::v2 a2 = cvt2<T>(v[4], v[5]), a3 = cvt2<T>(v[6], v[7]);
        V8 w = {a0[0], a0[1], a1[0], a1[1], a2[0], a2[1], a3[0], a3[1]};
        pf[2 * c + hh][j] = w;
      }

  // ---- second convolution (1x1): 32 output channels at a time, W2 rows from global
  const long long plane = (long long)p.P * p.Q;
  for (int ct = 0; ct * 32 < p.C2; ++ct) {
    const int c2row = 32 * ct + ln;  // A operand row of this lane
    f32x16 o[PXW];
#pragma unroll
    for (int j = 0; j < PXW; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[j][r] = 0.f;
#pragma unroll
    for (int u = 0; u < 2 * C1T; ++u) {
      V4 lo = {zero, zero, zero, zero}, hi = {zero, zero, zero, zero};
      const int k0 = 16 * u + 4 * g;
      if (c2row < p.C2) {
        const T* wr = W2g + (long long)c2row * p.C1;
        if (k0 + 3 < p.C1) lo = *reinterpret_cast<const V4*>(wr + k0);
        if (k0 + 8 + 3 < p.C1) hi = *reinterpret_cast<const V4*>(wr + k0 + 8);
      }
      const V8 wf = concat4<V4, V8>(lo, hi);
#pragma unroll
      for (int j = 0; j < PXW; ++j) o[j] = Elem<T>::mfma32(wf, pf[u][j], o[j]);
    }
    // o[j][r] = out^T[c2 = 32ct + 8(r/4) + 4g + r%4][pixel of lane]: for one r the 32 lanes of
    // a half-wave write consecutive pixels of one channel plane
#pragma unroll
    for (int j = 0; j < PXW; ++j) {
      if (!valid[j]) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c2 = 32 * ct + 8 * (r >> 2) + 4 * g + (r & 3);
        if (c2 >= p.C2) continue;
        float v = o[j][r];
        if (p.relu_out) v = fmaxf(v, 0.f);
        const long long off = ((long long)n * p.C2 + c2) * plane + opix[j];
        if (p.out_f32)
          reinterpret_cast<float*>(p.y)[off] = v;
        else
          reinterpret_cast<T*>(p.y)[off] = (T)v;
      }
    }
  }
}

template <typename T, int C1T, int PXW>
hipError_t launch_conv_chain(const ConvChainArgs& args, hipStream_t stream) {
  const int lds = conv_chain_lds_bytes(args.rows_in, args.cols_in, args.R * args.S, 32 * C1T);
  auto kern = conv_chain_kernel<T, C1T, PXW>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  const unsigned grid = (unsigned)args.N * (unsigned)args.tiles_h * (unsigned)args.tiles_w;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, args);
  return hipGetLastError();
}

}  // namespace ditto
