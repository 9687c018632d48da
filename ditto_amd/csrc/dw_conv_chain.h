// Fused depthwise conv(RxS, `mult` outputs per input channel) -> cast|relu -> conv(1x1) chain on
// NCHW tensors, fp16 / bf16, gfx950.
//
// Reference chain: benchmark/chimera/cuda/depthwise3x3_conv1x1_small_channel_cuda.py:77-169
// (`factor` = mult; the reference pads the 9 taps to a 16-deep tensor-core GEMM).  Here the
// depthwise stage runs on the VALU -- 9 multiply-adds per intermediate value, two at a time with
// v_dot2_f32_{f16,bf16} (fp32 accumulation) -- and produces the second contraction's MFMA operand
// directly: lane (pixel n, half g) computes the 8 consecutive intermediate channels
// 16*ks + 8*g .. +7 of its pixel, which is the B-operand fragment of k step ks of
//     out^T[c2][pix] = sum_cm W2[c2][cm] * mid[cm][pix].
// The intermediate exists only in registers.
//
// A workgroup (4 waves, 64 pixels each) owns TH x TW output pixels of one image and all output
// channels; input channels are walked in chunks: the halo tile of the chunk in its natural
// [channel][row][col] order, the chunk's depthwise filters as tap pairs and the matching columns
// of W2 are staged in LDS.
#pragma once
#include "common.h"

namespace ditto {

struct DwConvArgs {
  const void* x;
  const void* w1;  // [C1][1][R][S]
  const void* w2;  // [C2][C1]
  void* y;
  int N, C0, H, W;
  int mult, C1, R, S, pad, stride;
  int C2;
  int P, Q;
  int TH, TW, tiles_h, tiles_w, rows_in, cols_in;
  int chx;  // input channels per staged chunk (chx * mult is a multiple of 16)
  int relu_mid, relu_out, out_f32;
};

constexpr int kDwPairs = 5;    // tap pairs per filter: R*S <= 9, padded with zeros
constexpr int kDwW1Str = 16;   // elements per staged filter (32 bytes: one 16-byte + one 4-byte read)

__host__ __device__ inline int dw_conv_lds_bytes(int chx, int mult, int rows_in, int cols_in, int C2p) {
  const int cm = chx * mult;
  return (chx * rows_in * cols_in + cm * kDwW1Str + C2p * (cm + 8)) * 2;
}

// SHARED: mult is a multiple of 8, so the 8 intermediate channels of a lane share one input channel
template <typename T, int C2T, int PXW, bool SHARED>
__global__ __launch_bounds__(256) void dw_conv_chain_kernel(DwConvArgs p) {
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  typedef typename Elem<T>::v2 V2;
  constexpr int C2p = 32 * C2T;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  const int CM = p.chx * p.mult;  // intermediate channels per chunk
  const int W2S = CM + 8;
  const int xplane = p.rows_in * p.cols_in;
  T* const Xs = reinterpret_cast<T*>(smem_raw);   // [chx][rows_in][cols_in]
  T* const W1s = Xs + ((p.chx * xplane + 7) & ~7); // [CM][16]: taps 0..8, zeros
  T* const W2s = W1s + CM * kDwW1Str;              // [C2p][CM + 8]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, g = lane >> 5;
  const int RS = p.R * p.S;
  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
  const int tiles = p.tiles_h * p.tiles_w;
  const int n = lid / tiles;
  const int th = (lid % tiles) / p.tiles_w, tw = (lid % tiles) % p.tiles_w;
  const int p0 = th * p.TH, q0 = tw * p.TW;
  const int h0 = p0 * p.stride - p.pad, w0 = q0 * p.stride - p.pad;
  const T* __restrict__ Xg = reinterpret_cast<const T*>(p.x) + (long long)n * p.C0 * p.H * p.W;
  const T* __restrict__ W1g = reinterpret_cast<const T*>(p.w1);
  const T* __restrict__ W2g = reinterpret_cast<const T*>(p.w2);
  const T zero = (T)0.f;

  int xoff[PXW];
  bool valid[PXW];
  int opix[PXW];
#pragma unroll
  for (int j = 0; j < PXW; ++j) {
    const int slot = 32 * (PXW * wave + j) + ln;
    const int ph = slot / p.TW, pw = slot % p.TW;
    valid[j] = ph < p.TH && (p0 + ph) < p.P && (q0 + pw) < p.Q;
    const int phc = valid[j] ? ph : 0, pwc = valid[j] ? pw : 0;
    xoff[j] = (phc * p.stride) * p.cols_in + pwc * p.stride;
    opix[j] = (p0 + phc) * p.Q + q0 + pwc;
  }
  // element offsets of the taps inside a halo plane, in pairs (taps past R*S alias tap 0 and meet
  // zero weights)
  int tap_off[2 * kDwPairs];
#pragma unroll
  for (int t = 0; t < 2 * kDwPairs; ++t) tap_off[t] = t < RS ? (t / p.S) * p.cols_in + (t % p.S) : 0;

  f32x16 o[C2T][PXW];
#pragma unroll
  for (int t = 0; t < C2T; ++t)
#pragma unroll
    for (int j = 0; j < PXW; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[t][j][r] = 0.f;

  const long long hw = (long long)p.H * p.W;
  for (int c0 = 0; c0 < p.C0; c0 += p.chx) {
    const int cm_base = c0 * p.mult;  // first intermediate channel of the chunk
    __syncthreads();
    // ---- halo tile, natural layout: a wave owns (channel, row) pairs, lanes run along w
    for (int cr = wave; cr < p.chx * p.rows_in; cr += 4) {
      const int c = cr / p.rows_in, ri = cr - c * p.rows_in;
      const int h = h0 + ri;
      const bool row_ok = c0 + c < p.C0 && h >= 0 && h < p.H;
      const T* src = Xg + (long long)(c0 + c) * hw + (long long)h * p.W;
      for (int ci = lane; ci < p.cols_in; ci += 64) {
        const int w = w0 + ci;
        Xs[c * xplane + ri * p.cols_in + ci] = (row_ok && w >= 0 && w < p.W) ? src[w] : zero;
      }
    }
    // ---- depthwise filters of the chunk: [cm][16], taps >= R*S zero
    for (int e = tid; e < CM * kDwW1Str; e += 256) {
      const int cm = e / kDwW1Str, t = e % kDwW1Str;
      W1s[e] = (t < RS && cm_base + cm < p.C1) ? W1g[(long long)(cm_base + cm) * RS + t] : zero;
    }
    // ---- the chunk's columns of W2: [c2][CM] (+8 pad), 16-byte vectors where the row allows
    for (int e = tid; e < C2p * (CM / 8); e += 256) {
      const int c2 = e / (CM / 8), v8 = e % (CM / 8);
      V8 v = {zero, zero, zero, zero, zero, zero, zero, zero};
      if (c2 < p.C2) {
        const T* src = W2g + (long long)c2 * p.C1 + cm_base + 8 * v8;
        if (cm_base + 8 * v8 + 7 < p.C1 && (p.C1 & 7) == 0) {
          v = *reinterpret_cast<const V8*>(src);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i)
            if (cm_base + 8 * v8 + i < p.C1) v[i] = src[i];
        }
      }
      *reinterpret_cast<V8*>(W2s + c2 * W2S + 8 * v8) = v;
    }
    __syncthreads();

    for (int ks = 0; ks * 16 < CM; ++ks) {
      const int cm0 = 16 * ks + 8 * g;  // chunk-relative first intermediate channel of this lane
      V8 pf[PXW];
#pragma unroll
      for (int j = 0; j < PXW; ++j) {
        float mid[8];
        V2 xp[kDwPairs];
        auto gather = [&](int c) __attribute__((always_inline)) {
          const T* xs = Xs + c * xplane + xoff[j];
#pragma unroll
          for (int q = 0; q < kDwPairs; ++q) xp[q] = V2{xs[tap_off[2 * q]], xs[tap_off[2 * q + 1]]};
        };
        if (SHARED) gather(cm0 / p.mult);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if (!SHARED) gather((cm0 + e) / p.mult);
          const T* wrow = W1s + (cm0 + e) * kDwW1Str;
          const V8 w8 = *reinterpret_cast<const V8*>(wrow);
          const V2 w4 = *reinterpret_cast<const V2*>(wrow + 8);
          float s = 0.f;
          s = Elem<T>::dot2(V2{w8[0], w8[1]}, xp[0], s);
          s = Elem<T>::dot2(V2{w8[2], w8[3]}, xp[1], s);
          s = Elem<T>::dot2(V2{w8[4], w8[5]}, xp[2], s);
          s = Elem<T>::dot2(V2{w8[6], w8[7]}, xp[3], s);
          s = Elem<T>::dot2(w4, xp[4], s);
          if (p.relu_mid) s = fmaxf(s, 0.f);
          mid[e] = s;
        }
        const V2 a0 = cvt2<T>(mid[0], mid[1]), a1 = cvt2<T>(mid[2], mid[3]);
        const V2 a2 = cvt2<T>(mid[4], mid[5]), a3 = cvt2<T>(mid[6], mid[7]);
        pf[j] = V8{a0[0], a0[1], a1[0], a1[1], a2[0], a2[1], a3[0], a3[1]};
      }
#pragma unroll
      for (int t = 0; t < C2T; ++t) {
        const V8 wf = *reinterpret_cast<const V8*>(W2s + (32 * t + ln) * W2S + cm0);
#pragma unroll
        for (int j = 0; j < PXW; ++j) o[t][j] = Elem<T>::mfma32(wf, pf[j], o[t][j]);
      }
    }
  }

  // o[t][j][r] = out^T[c2 = 32t + 8(r/4) + 4g + r%4][pixel of lane]
  const long long plane = (long long)p.P * p.Q;
#pragma unroll
  for (int t = 0; t < C2T; ++t)
#pragma unroll
    for (int j = 0; j < PXW; ++j) {
      if (!valid[j]) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int c2 = 32 * t + 8 * (r >> 2) + 4 * g + (r & 3);
        if (c2 >= p.C2) continue;
        float v = o[t][j][r];
        if (p.relu_out) v = fmaxf(v, 0.f);
        const long long off = ((long long)n * p.C2 + c2) * plane + opix[j];
        if (p.out_f32)
          reinterpret_cast<float*>(p.y)[off] = v;
        else
          reinterpret_cast<T*>(p.y)[off] = (T)v;
      }
    }
}

template <typename T, int C2T, int PXW, bool SHARED>
hipError_t launch_dw_conv_chain(const DwConvArgs& args, hipStream_t stream) {
  const int lds = dw_conv_lds_bytes(args.chx, args.mult, args.rows_in, args.cols_in, 32 * C2T) + 16;
  auto kern = dw_conv_chain_kernel<T, C2T, PXW, SHARED>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  const unsigned grid = (unsigned)args.N * (unsigned)args.tiles_h * (unsigned)args.tiles_w;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, args);
  return hipGetLastError();
}

}  // namespace ditto
