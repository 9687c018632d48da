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
#include <type_traits>

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
  int chx;  // input channels per staged chunk (chx * mult is a multiple of 16; 32 on the MFMA path)
  int relu_mid, relu_out, out_f32;
  // MFMA path
  int vec;      // elements per halo load (1, 2, 4): divides W, x is aligned to 2 * vec bytes
  int cols_al;  // LDS row stride of the halo tile: cols_in + vec - 1 rounded up to vec
  int wide;     // 16-byte output stores through LDS: Q and TW multiples of 8, y 16-byte aligned, not fp32
  int grid;     // persistent workgroups
  int nt_store; // WIDE: streaming (non-temporal) output stores
};

constexpr int kDwPairs = 5;    // tap pairs per filter: R*S <= 9, padded with zeros
constexpr int kDwW1Str = 16;   // elements per staged filter (32 bytes: one 16-byte + one 4-byte read)

__host__ __device__ inline int dw_conv_lds_bytes(int chx, int mult, int rows_in, int cols_in, int C2p) {
  const int cm = chx * mult;
  return (chx * rows_in * cols_in + cm * kDwW1Str + C2p * (cm + 8)) * 2;
}

// Halo tile of input channels c0 .. c0+chx-1 into Xs[chx][rows_in][cols_in]: threads form
// (256 / LW) row slots x LW columns, LW the power of two covering cols_in (at most 64); eight
// 2-byte loads are in flight per thread before their LDS stores.
template <typename T>
__device__ __forceinline__ void stage_halo(T* __restrict__ Xs, const T* __restrict__ Xg, const DwConvArgs& p, int c0,
                                           int h0, int w0, int tid) {
  int lw_shift = 3;
  while ((1 << lw_shift) < p.cols_in && lw_shift < 6) ++lw_shift;
  const int LW = 1 << lw_shift, rpp = 256 >> lw_shift;
  const int col = tid & (LW - 1), rslot = tid >> lw_shift;
  const int nrows = p.chx * p.rows_in;
  const int xplane = p.rows_in * p.cols_in;
  const long long hw = (long long)p.H * p.W;
  // (rowid + 0.5) / rows_in in fp32 floors to the exact quotient: the quotient is below
  // 80K / rows_in (the tile fits in LDS), so the rounding error stays under 0.02 / rows_in
  const float inv_rows = 1.0f / (float)p.rows_in;
  const T zero = (T)0.f;
  for (int cseg = 0; cseg < p.cols_in; cseg += LW) {
    const int ci = cseg + col, w = w0 + ci;
    const bool col_ok = ci < p.cols_in, w_ok = col_ok && w >= 0 && w < p.W;
    for (int base = rslot; base < nrows; base += 8 * rpp) {
      T v[8];
      int dst[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int rowid = base + u * rpp;
        const int c = (int)(((float)rowid + 0.5f) * inv_rows);
        const int ri = rowid - c * p.rows_in;
        const int h = h0 + ri;
        dst[u] = (rowid < nrows && col_ok) ? c * xplane + ri * p.cols_in + ci : -1;
        v[u] = zero;
        if (dst[u] >= 0 && w_ok && c0 + c < p.C0 && h >= 0 && h < p.H)
          v[u] = Xg[(long long)(c0 + c) * hw + (long long)h * p.W + w];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (dst[u] >= 0) Xs[dst[u]] = v[u];
    }
  }
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
    wg_sync();
    // ---- halo tile, natural layout: a wave owns (channel, row) pairs, lanes run along w
    stage_halo<T>(Xs, Xg, p, c0, h0, w0, tid);
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
    wg_sync();

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

// ---------------------------------------------------------------------------------------------
// Channel multipliers that are multiples of 16: the depthwise stage on the matrix cores as well.
// One 32x32x16 MFMA produces 32 intermediate channels x 32 pixels from two 8-deep halves:
//     rows 0..15  (intermediate channels cmb .. cmb+15)  contract over k = 0..7,
//     rows 16..31 (intermediate channels cmb+16 .. +31)  contract over k = 8..15,
// a block-diagonal A operand (the filters' taps 0..7, zeros in the other half), with the B operand
// of lane (pixel n, half g) holding taps 0..7 of the input channel that owns rows 16g..16g+15.
// Taps 8.. (the ninth of a 3x3 filter) go through a second MFMA of the same form.  Rows are
// assigned to intermediate channels so that the accumulator registers 8s..8s+7 of lane (n, g)
// are the consecutive channels cmb + 16s + 8g .. +7: converted, they are the operand of k step s
// of the 1x1 convolution against W2 in its natural layout.
//
// Workgroups are persistent: each walks pixel tiles lid, lid + grid, ... with 4 * NG waves (eight
// where the registers allow, so that every SIMD has two waves to issue from); pixel tiles of 32
// go to the waves round-robin.  When all input channels fit in one chunk the filters
// are staged once per workgroup and stay in LDS; the halo tile of the next (tile, chunk) is
// loaded into registers while the current one is computed.
//
// LDS:  Xs  [chx][rows_in][cols_al]            halo tile; columns start at the tile's first column
//                                            rounded down to the load width, so rows are stored
//                                            with the vectors they were loaded with
//       W1h [CM / 32][2][32] x 16 bytes      taps 0..7 | 8..15 of the 32 rows of each block, then
//                                            one zero entry (the other half of the block diagonal)
//       W2s [32 * C2T][CM + 8]               the chunk's columns of W2
//       Os  [waves][32][40]                  WIDE: per-wave turn-around for 16-byte stores
constexpr int kDwMfmaTaps = 16;  // R * S <= 16 on the MFMA path
constexpr int kDwXpf = 12;      // halo vectors of up to 4 elements (or half as many of 8) a thread keeps in flight

constexpr int kDwOss = 40;  // row stride (elements) of a wave's turn-around buffer: 32 pixels + 8

// tile shape of the MFMA path per output-channel tile count: pixel tiles per wave and waves / 4 per
// workgroup (register budget: two waves per SIMD leave 256 registers each)
__host__ __device__ constexpr int dw_mfma_pxw(int c2_tiles) { return 1; }
__host__ __device__ constexpr int dw_mfma_groups(int c2_tiles) { return c2_tiles <= 2 ? 2 : 1; }

__host__ __device__ inline int dw_conv_mfma_lds_bytes(int chx, int mult, int rows_in, int cols_al, int C2p,
                                                      int groups, bool wide) {
  const int cm = chx * mult;
  return ((chx * rows_in * cols_al + 7) & ~7) * 2 + ((cm / 32) * 64 + 1) * 16 + C2p * (cm + 8) * 2 +
         (wide ? 4 * groups * 32 * kDwOss * 2 : 0);
}

template <typename T, int VEC>
__device__ __forceinline__ void dw_ld_vec(typename Elem<T>::v4& r, const T* src) {
  if constexpr (VEC == 4) {
    r = *reinterpret_cast<const typename Elem<T>::v4*>(src);
  } else if constexpr (VEC == 2) {
    const typename Elem<T>::v2 t = *reinterpret_cast<const typename Elem<T>::v2*>(src);
    r[0] = t[0]; r[1] = t[1];
  } else {
    r[0] = *src;
  }
}

// 8-element (16-byte) halo vectors occupy two consecutive entries of the register array
template <typename T>
__device__ __forceinline__ void dw_ld_vec8(typename Elem<T>::v4& lo, typename Elem<T>::v4& hi, const T* src) {
  const typename Elem<T>::v8 t = *reinterpret_cast<const typename Elem<T>::v8*>(src);
  lo = typename Elem<T>::v4{t[0], t[1], t[2], t[3]};
  hi = typename Elem<T>::v4{t[4], t[5], t[6], t[7]};
}
template <typename T>
__device__ __forceinline__ void dw_st_vec8(T* dst, const typename Elem<T>::v4& lo, const typename Elem<T>::v4& hi) {
  *reinterpret_cast<typename Elem<T>::v8*>(dst) = typename Elem<T>::v8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
}

template <typename T, int VEC>
__device__ __forceinline__ void dw_st_vec(T* dst, const typename Elem<T>::v4& r) {
  if constexpr (VEC == 4) {
    *reinterpret_cast<typename Elem<T>::v4*>(dst) = r;
  } else if constexpr (VEC == 2) {
    *reinterpret_cast<typename Elem<T>::v2*>(dst) = typename Elem<T>::v2{r[0], r[1]};
  } else {
    *dst = r[0];
  }
}

// F33: 3x3 filter.  The nine taps of a pixel are then gathered with one two-dword LDS read per
// filter row (the dword pair that covers columns w .. w+2) and funnel shifts by the pixel's column
// parity, and sit in the operand in the order r0s0 r0s1 r1s0 r1s1 r2s0 r2s1 r0s2 r1s2 | r2s2; other
// filters gather tap by tap in their natural order.
__host__ __device__ constexpr int dw_tap_of_k(bool f33, int k) {
  return !f33 ? k : k == 0 ? 0 : k == 1 ? 1 : k == 2 ? 3 : k == 3 ? 4 : k == 4 ? 6 : k == 5 ? 7 : k == 6 ? 2 : k == 7 ? 5 : k;
}

//
// DWV (3x3 filters, channel multiplier 1, 2, 4 or 8): the same persistent kernel with the depthwise
// stage on the vector ALU -- a block-diagonal MFMA would use mult of every 16 rows.  A lane gathers
// the taps of its pixel as above (once per input channel it needs) and takes five
// v_dot2_f32_f16/bf16 per intermediate value against the filter's tap pairs, kept in LDS in the
// same order: entry 2 * cm holds pairs 0..3, entry 2 * cm + 1 the ninth tap.
// MSH = log2(multiplier) there (a compile-time constant keeps the gather-sharing pattern static);
// -1: the matrix-core depthwise stage.
template <typename T, int C2T, int PXW, int NG, bool WIDE, bool F33, int MSH = -1>
__global__ __launch_bounds__(256 * NG) void dw_conv_mfma_kernel(DwConvArgs p) {
  constexpr bool DWV = MSH >= 0;
  static_assert(!DWV || (F33 && WIDE), "the vector-ALU depthwise stage is built for 3x3 filters and 16-byte stores");
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  typedef typename Elem<T>::v2 V2;
  constexpr int C2p = 32 * C2T;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  const int CM = p.chx * p.mult, nblk = CM / 32;
  const int W2S = CM + 8;
  const int xplane = p.rows_in * p.cols_al;
  const int xs_elems = (p.chx * xplane + 7) & ~7;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int NT = 256 * NG, NW = 4 * NG;  // threads, waves of the workgroup
  const int ln = lane & 31, g = lane >> 5;
  T* const Xs = reinterpret_cast<T*>(smem_raw);
  uint4* const W1h = reinterpret_cast<uint4*>(Xs + xs_elems);
  T* const W2s = reinterpret_cast<T*>(W1h + nblk * 64 + 1);
  T* const Ow = W2s + C2p * W2S + wave * 32 * kDwOss;  // this wave's turn-around buffer

  const int RS = p.R * p.S;
  const bool second_half = F33 || RS > 8;
  const T* __restrict__ Xg = reinterpret_cast<const T*>(p.x);
  const T* __restrict__ W1g = reinterpret_cast<const T*>(p.w1);
  const T* __restrict__ W2g = reinterpret_cast<const T*>(p.w2);
  const T zero = (T)0.f;
  const V8 zero8 = {zero, zero, zero, zero, zero, zero, zero, zero};
  const int npix_tiles = (p.TH * p.TW + 31) / 32;  // pixel tiles of a workgroup's tile that hold pixels
  const long long hw = (long long)p.H * p.W;
  const long long plane = (long long)p.P * p.Q;
  const int tiles = p.tiles_h * p.tiles_w;
  const int ntiles = p.N * tiles;
  const int nchunks = (p.C0 + p.chx - 1) / p.chx;
  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);

  // ---- halo staging: a thread owns one (row, vector) position of the halo tile and walks the
  // chunk's channels: thread tid = slot * nvr + vi with slot = cph * rows_in + ri; pass u brings
  // channel cph + u * cphases.  Addresses advance by constants from pass to pass and the row /
  // column bounds are tested once per tile.  (The host sizes chunks so that kDwXpf passes cover them.)
  const int nvr = p.cols_al / p.vec;
  const int cphases = (NT / nvr) / p.rows_in;  // >= 1: checked by the host
  const int st_slot = tid / nvr, st_vi = tid - st_slot * nvr;
  const int st_cph = st_slot / p.rows_in, st_ri = st_slot - st_cph * p.rows_in;
  const bool st_on = st_cph < cphases;
  const int st_dst = st_cph * xplane + st_ri * p.cols_al + st_vi * p.vec;
  const int hw32 = p.H * p.W;
  V4 xr[kDwXpf];
  const V4 zero4 = {zero, zero, zero, zero};
  // halo vectors of chunk c0 of tile `tile` into registers
  auto xload = [&](int tile, int c0) __attribute__((always_inline)) {
    const int n = tile / tiles, rem = tile - n * tiles;
    const int th = rem / p.tiles_w, tw = rem - th * p.tiles_w;
    const int h = th * p.TH * p.stride - p.pad + st_ri;
    const int w = ((tw * p.TW * p.stride - p.pad) & ~(p.vec - 1)) + st_vi * p.vec;
    const bool ok = st_on && h >= 0 && h < p.H && w >= 0 && w < p.W;
    const int nch = (p.C0 - c0 < p.chx ? p.C0 - c0 : p.chx) - st_cph;  // channels left for this thread
    const long long src = ((long long)n * p.C0 + c0 + st_cph) * hw + (long long)h * p.W + w;
    auto body = [&](auto vec_tag) __attribute__((always_inline)) {
      constexpr int VEC = decltype(vec_tag)::value;
      // a running element offset: per-pass offsets would be hoisted out of the tile loop and spilled
      // (an offset and not a pointer: a pointer that has passed through the asm below is no longer
      // known to point to global memory)
      long long q = src;
      int left = nch;
      if constexpr (VEC == 8) {
#pragma unroll
        for (int u = 0; u < kDwXpf / 2; ++u) {
          xr[2 * u] = zero4;
          xr[2 * u + 1] = zero4;
          if (ok && left > 0) dw_ld_vec8<T>(xr[2 * u], xr[2 * u + 1], Xg + q);
          q += cphases * hw32;
          left -= cphases;
          asm volatile("" : "+v"(q), "+v"(left));
        }
        return;
      }
#pragma unroll
      for (int u = 0; u < kDwXpf; ++u) {
        xr[u] = zero4;
        if (ok && left > 0) dw_ld_vec<T, VEC>(xr[u], Xg + q);
        q += cphases * hw32;
        left -= cphases;
        asm volatile("" : "+v"(q), "+v"(left));
      }
    };
    if (p.vec == 8) body(std::integral_constant<int, 8>());
    else if (p.vec == 4) body(std::integral_constant<int, 4>());
    else if (p.vec == 2) body(std::integral_constant<int, 2>());
    else body(std::integral_constant<int, 1>());
  };
  auto xstore = [&]() __attribute__((always_inline)) {
    auto body = [&](auto vec_tag) __attribute__((always_inline)) {
      constexpr int VEC = decltype(vec_tag)::value;
      int q = st_dst;  // a running offset, as in xload (a pointer would no longer be known to point to LDS)
      int left = st_on ? p.chx - st_cph : 0;
      if constexpr (VEC == 8) {
#pragma unroll
        for (int u = 0; u < kDwXpf / 2; ++u) {
          if (left > 0) dw_st_vec8<T>(Xs + q, xr[2 * u], xr[2 * u + 1]);
          q += cphases * xplane;
          left -= cphases;
          asm volatile("" : "+v"(q), "+v"(left));
        }
        return;
      }
#pragma unroll
      for (int u = 0; u < kDwXpf; ++u) {
        if (left > 0) dw_st_vec<T, VEC>(Xs + q, xr[u]);
        q += cphases * xplane;
        left -= cphases;
        asm volatile("" : "+v"(q), "+v"(left));
      }
    };
    if (p.vec == 8) body(std::integral_constant<int, 8>());
    else if (p.vec == 4) body(std::integral_constant<int, 4>());
    else if (p.vec == 2) body(std::integral_constant<int, 2>());
    else body(std::integral_constant<int, 1>());
  };

  // ---- pixel slots of this lane (the same in every tile): pixel tiles go to the waves round-robin
  int xoff[PXW], sph[PXW], spw[PXW];
#pragma unroll
  for (int j = 0; j < PXW; ++j) {
    const int slot = 32 * (wave + NW * j) + ln;
    const int ph = slot / p.TW, pw = slot - ph * p.TW;
    const bool in_tile = ph < p.TH;
    sph[j] = in_tile ? ph : -1;
    spw[j] = pw;
    xoff[j] = in_tile ? (ph * p.stride) * p.cols_al + pw * p.stride : 0;
  }
  // WIDE output: vector v = 64i + lane of a pixel tile is (channel v / 4, 8 pixels from slot
  // 8 * (lane % 4)); the row / column of that slot inside the workgroup's tile are the same in every tile
  int ov_ph[PXW], ov_pw[PXW];
#pragma unroll
  for (int j = 0; j < PXW; ++j) {
    const int slot = 32 * (wave + NW * j) + 8 * (lane & 3);
    const int ph = slot / p.TW;
    ov_ph[j] = ph < p.TH ? ph : 1 << 20;  // past the tile: fails the row test below
    ov_pw[j] = slot - ph * p.TW;
  }
  int tap_off[kDwMfmaTaps];
#pragma unroll
  for (int t = 0; t < kDwMfmaTaps; ++t) tap_off[t] = (!F33 && t < RS) ? (t / p.S) * p.cols_al + (t % p.S) : 0;
  // A-operand entry of this lane inside a block: its own half of the block diagonal, else zeros
  const bool own_half = (ln >> 4) == g;
  const int zero_entry = nblk * 64;
  const float inv_m16 = 16.0f / (float)p.mult;

  if ((int)lid < ntiles) xload((int)lid, 0);
  bool weights_staged = false;
  for (int tile = (int)lid; tile < ntiles; tile += (int)gridDim.x) {
    const int tile_next = tile + (int)gridDim.x < ntiles ? tile + (int)gridDim.x : -1;
    const int n = tile / tiles, rem = tile - n * tiles;
    const int th = rem / p.tiles_w, tw = rem - th * p.tiles_w;
    const int p0 = th * p.TH, q0 = tw * p.TW;
    const int w0 = q0 * p.stride - p.pad;
    const int lead = w0 - (w0 & ~(p.vec - 1));

    f32x16 o[C2T][PXW];
#pragma unroll
    for (int t = 0; t < C2T; ++t)
#pragma unroll
      for (int j = 0; j < PXW; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[t][j][r] = 0.f;

    for (int chunk = 0; chunk < nchunks; ++chunk) {
      const int c0 = chunk * p.chx;
      const int cm_base = c0 * p.mult;
      wg_sync();  // every wave is done with the previous halo tiles (and filters, if restaged)
      xstore();
      if (!weights_staged || nchunks > 1) {
        weights_staged = true;
        // the chunk's depthwise filters, CM * RS contiguous elements, pass through the W2 area (16-byte
        // loads; C1 * RS is a multiple of 8 and the chunk starts on a 16-byte boundary) ...
        {
          const long long first = (long long)cm_base * RS, total = (long long)p.C1 * RS;
          for (int e = tid; e * 8 < CM * RS; e += NT) {
            V8 v = zero8;
            if (first + 8 * e < total) v = *reinterpret_cast<const V8*>(W1g + first + 8 * e);
            *reinterpret_cast<V8*>(W2s + 8 * e) = v;
          }
        }
        wg_sync();
        // ... and are regrouped into A-operand entries: row m = 16 * hgrp + 8a + 4gg + b of a block is
        // its intermediate channel 16 * hgrp + 8gg + 4a + b (DWV: two entries per intermediate channel)
        for (int e = tid; e < nblk * 64; e += NT) {
          const int m = e & 31, half = DWV ? (e & 1) : ((e >> 5) & 1), blk = e >> 6;
          if (half && !second_half) continue;
          const int mm = m & 15;
          const int cml = DWV ? (e >> 1)
                              : 32 * blk + 16 * (m >> 4) + 8 * ((mm >> 2) & 1) + 4 * (mm >> 3) + (mm & 3);
          unsigned raw[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int tap = dw_tap_of_k(F33, 8 * half + i);
            raw[i] = tap < RS ? reinterpret_cast<const unsigned short*>(W2s)[cml * RS + tap] : 0;
          }
          W1h[e] = uint4{raw[0] | (raw[1] << 16), raw[2] | (raw[3] << 16), raw[4] | (raw[5] << 16),
                         raw[6] | (raw[7] << 16)};
        }
        if (tid == 0) W1h[zero_entry] = uint4{0, 0, 0, 0};
        wg_sync();
        const int nv = CM / 8;  // 16-byte vectors per row of the W2 chunk (C1 is a multiple of 16 here)
        const float inv_nv = 1.0f / (float)nv;
        for (int e0 = tid; e0 < C2p * nv; e0 += 4 * NT) {
          V8 v[4];
          int dst[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int e = e0 + NT * u;
            const int c2 = (int)(((float)e + 0.5f) * inv_nv);  // exact: e < 2^21, the quotient below 2^9
            const int v8 = e - c2 * nv;
            dst[u] = e < C2p * nv ? c2 * W2S + 8 * v8 : -1;
            v[u] = zero8;
            if (dst[u] >= 0 && c2 < p.C2 && cm_base + 8 * v8 < p.C1)
              v[u] = *reinterpret_cast<const V8*>(W2g + (long long)c2 * p.C1 + cm_base + 8 * v8);
          }
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (dst[u] >= 0) *reinterpret_cast<V8*>(W2s + dst[u]) = v[u];
        }
      }
      wg_sync();
      // the next (tile, chunk) travels while this one is computed
      if (chunk + 1 < nchunks) xload(tile, c0 + p.chx);
      else if (tile_next >= 0) xload(tile_next, 0);

      // Software pipeline over units (block of 32 intermediate channels, pixel tile): while the
      // 1x1 convolution consumes unit U (operand pf already converted), the depthwise result of
      // unit U+1 is in flight in `acc`; after the MFMAs of U have issued it is converted and the
      // depthwise MFMAs of unit U+2 start, so every MFMA result has the next unit's MFMAs to
      // mature under.  One accumulator and one operand per pixel tile are live.  W2 fragments of
      // the next block are read once the last MFMA that uses the current ones has issued.  Units
      // past the end recompute the last block and are discarded.
      V8 a1n, a2n, b1n, b2n, wf[C2T][2], pf[PXW][2];
      f32x16 acc;
      auto load_w2 = [&](int blk) __attribute__((always_inline)) {
#pragma unroll
        for (int t = 0; t < C2T; ++t)
#pragma unroll
          for (int s = 0; s < 2; ++s)
            wf[t][s] = *reinterpret_cast<const V8*>(W2s + (32 * t + ln) * W2S + 32 * blk + 16 * s + 8 * g);
      };
      auto load_a = [&](int blk) __attribute__((always_inline)) {
        a1n = __builtin_bit_cast(V8, W1h[own_half ? (2 * blk) * 32 + ln : zero_entry]);
        a2n = __builtin_bit_cast(V8, W1h[(own_half && second_half) ? (2 * blk + 1) * 32 + ln : zero_entry]);
      };
      auto load_b = [&](int blk, int j) __attribute__((always_inline)) {
        // input channel (chunk-relative) behind rows 16g .. 16g+15 of the block; the fp32 quotient
        // is exact for these small numbers
        const int c = (int)(((float)(2 * blk + g) + 0.5f) * inv_m16);
        if constexpr (F33) {
          // dword pair (4 elements) from the even column at or below the pixel's first tap column
          const int xc = xoff[j] + lead;
          const unsigned* xw = reinterpret_cast<const unsigned*>(Xs + c * xplane + (xc & ~1));
          const unsigned sh = (xc & 1) * 16;
          unsigned p01[3], t2[3];
#pragma unroll
          for (int r = 0; r < 3; ++r) {
            const unsigned d0 = xw[r * (p.cols_al >> 1)], d1 = xw[r * (p.cols_al >> 1) + 1];
            p01[r] = __builtin_amdgcn_alignbit(d1, d0, sh);  // columns w, w+1
            t2[r] = __builtin_amdgcn_alignbit(0u, d1, sh);   // column w+2 in the low half
          }
          const uint4 b1r = {p01[0], p01[1], p01[2], __builtin_amdgcn_perm(t2[1], t2[0], 0x05040100u)};
          const uint4 b2r = {t2[2] & 0xffffu, 0u, 0u, 0u};
          b1n = __builtin_bit_cast(V8, b1r);
          b2n = __builtin_bit_cast(V8, b2r);
        } else {
          const T* xs = Xs + c * xplane + xoff[j] + lead;
          b1n = V8{xs[tap_off[0]], xs[tap_off[1]], xs[tap_off[2]], xs[tap_off[3]],
                   xs[tap_off[4]], xs[tap_off[5]], xs[tap_off[6]], xs[tap_off[7]]};
          b2n = V8{xs[tap_off[8]], zero, zero, zero, zero, zero, zero, zero};
          if (RS > 9) {  // taps past R * S alias tap 0 and meet zero filter entries
#pragma unroll
            for (int i = 1; i < 8; ++i) b2n[i] = xs[tap_off[8 + i]];
          }
        }
      };
      auto depthwise = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f;
        acc = Elem<T>::mfma32(a1n, b1n, acc);
        if (second_half) acc = Elem<T>::mfma32(a2n, b2n, acc);
      };
      auto convert = [&](int j) __attribute__((always_inline)) {
        if (p.relu_mid) {
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[r] = fmaxf(acc[r], 0.f);
        }
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          const V2 c0v = cvt2<T>(acc[8 * s + 0], acc[8 * s + 1]), c1v = cvt2<T>(acc[8 * s + 2], acc[8 * s + 3]);
          const V2 c2v = cvt2<T>(acc[8 * s + 4], acc[8 * s + 5]), c3v = cvt2<T>(acc[8 * s + 6], acc[8 * s + 7]);
          pf[j][s] = V8{c0v[0], c0v[1], c1v[0], c1v[1], c2v[0], c2v[1], c3v[0], c3v[1]};
        }
      };
      auto pointwise = [&](int j) __attribute__((always_inline)) {
        if (wave + NW * j < npix_tiles) {  // wave-uniform
#pragma unroll
          for (int t = 0; t < C2T; ++t) {
            if (WIDE) {  // pixel-major result: rows = pixels, columns = output channels
              o[t][j] = Elem<T>::mfma32(pf[j][0], wf[t][0], o[t][j]);
              o[t][j] = Elem<T>::mfma32(pf[j][1], wf[t][1], o[t][j]);
            } else {
              o[t][j] = Elem<T>::mfma32(wf[t][0], pf[j][0], o[t][j]);
              o[t][j] = Elem<T>::mfma32(wf[t][1], pf[j][1], o[t][j]);
            }
          }
        }
      };
      const int last = nblk - 1;
      if constexpr (DWV) {
        constexpr int msh = DWV ? MSH : 0;  // log2 of the channel multiplier
        const int row_dw = p.cols_al >> 1;  // dwords per halo row (cols_al is even here)
        for (int blk = 0; blk < nblk; ++blk) {
          load_w2(blk);
#pragma unroll
          for (int j = 0; j < PXW; ++j) {
            const int xc = xoff[j] + lead;
            const unsigned sh = (xc & 1) * 16;
            // Element offset of the lane's part of every gather address below, made opaque here:
            // the rest of each address (input channel and halo row) is the same in every lane and
            // stays in scalar registers.  Left to itself the compiler keeps one vector register
            // per address for the whole kernel plus one per address and tile; that does not fit,
            // and every reload from scratch waits for all outstanding output stores.
            int xlane = ((8 * g) >> msh) * xplane + (xc & ~1);
            asm volatile("" : "+v"(xlane));
#pragma unroll
            for (int s = 0; s < 2; ++s) {
              const int cu0 = 32 * blk + 16 * s;          // the lane-independent part of cm0
              const int cm0 = cu0 + 8 * g;                // first of the lane's 8 intermediate channels
              unsigned tp[5] = {0, 0, 0, 0, 0};           // tap pairs of the current input channel
              float mid[8];
#pragma unroll
              for (int e = 0; e < 8; ++e) {
                if ((e & ((1 << msh) - 1)) == 0) {  // a new input channel starts
                  // (cm0 + e) >> msh = ((cu0 + e) >> msh) + ((8 * g) >> msh): cu0 is a multiple of 16
                  const unsigned* xw =
                      reinterpret_cast<const unsigned*>(Xs + (xlane + ((cu0 + e) >> msh) * xplane));
                  unsigned t2[3];
#pragma unroll
                  for (int r = 0; r < 3; ++r) {
                    const unsigned d0 = xw[r * row_dw], d1 = xw[r * row_dw + 1];
                    tp[r] = __builtin_amdgcn_alignbit(d1, d0, sh);
                    t2[r] = __builtin_amdgcn_alignbit(0u, d1, sh);
                  }
                  tp[3] = __builtin_amdgcn_perm(t2[1], t2[0], 0x05040100u);
                  tp[4] = t2[2] & 0xffffu;
                }
                const uint4 w = W1h[2 * (cm0 + e)];
                const unsigned w8 = W1h[2 * (cm0 + e) + 1].x;
                float a = Elem<T>::dot2(__builtin_bit_cast(V2, w.x), __builtin_bit_cast(V2, tp[0]), 0.f);
                a = Elem<T>::dot2(__builtin_bit_cast(V2, w.y), __builtin_bit_cast(V2, tp[1]), a);
                a = Elem<T>::dot2(__builtin_bit_cast(V2, w.z), __builtin_bit_cast(V2, tp[2]), a);
                a = Elem<T>::dot2(__builtin_bit_cast(V2, w.w), __builtin_bit_cast(V2, tp[3]), a);
                a = Elem<T>::dot2(__builtin_bit_cast(V2, w8), __builtin_bit_cast(V2, tp[4]), a);
                mid[e] = p.relu_mid ? fmaxf(a, 0.f) : a;
              }
              const V2 c0v = cvt2<T>(mid[0], mid[1]), c1v = cvt2<T>(mid[2], mid[3]);
              const V2 c2v = cvt2<T>(mid[4], mid[5]), c3v = cvt2<T>(mid[6], mid[7]);
              pf[j][s] = V8{c0v[0], c0v[1], c1v[0], c1v[1], c2v[0], c2v[1], c3v[0], c3v[1]};
            }
            pointwise(j);
          }
        }
      } else {
      load_a(0);
      load_w2(0);
      load_b(0, 0);
      depthwise();
      convert(0);
      if constexpr (PXW == 2) {
        load_b(0, 1);
        depthwise();
        for (int blk = 0; blk < nblk; ++blk) {
          const int nxt = blk < last ? blk + 1 : last;
          load_a(nxt);
          load_b(nxt, 0);
          __builtin_amdgcn_sched_barrier(0);
          pointwise(0);
          __builtin_amdgcn_sched_barrier(0);
          convert(1);  // unit (blk, 1)
          depthwise();  // unit (nxt, 0)
          load_b(nxt, 1);
          __builtin_amdgcn_sched_barrier(0);
          pointwise(1);
          __builtin_amdgcn_sched_barrier(0);
          load_w2(nxt);
          convert(0);  // unit (nxt, 0)
          depthwise();  // unit (nxt, 1)
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        load_a(last < 1 ? last : 1);
        load_b(last < 1 ? last : 1, 0);
        depthwise();
        for (int blk = 0; blk < nblk; ++blk) {
          const int nxt = blk < last ? blk + 1 : last, nx2 = blk + 2 < last ? blk + 2 : last;
          load_a(nx2);
          load_b(nx2, 0);
          __builtin_amdgcn_sched_barrier(0);
          pointwise(0);
          __builtin_amdgcn_sched_barrier(0);
          load_w2(nxt);
          convert(0);   // unit nxt
          depthwise();  // unit nx2
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      }
    }
    if (WIDE) {
      // o[t][j][r] = out[pixel 8(r/4) + 4g + r%4 of tile j][c2 = 32t + ln]: four consecutive pixels of
      // one channel per register quad -> 8-byte LDS writes into this wave's corner, 16-byte stores out
#pragma unroll
      for (int t = 0; t < C2T; ++t)
#pragma unroll
        for (int j = 0; j < PXW; ++j) {
          if (wave + NW * j >= npix_tiles) continue;  // wave-uniform
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              v[e] = o[t][j][4 * q + e];
              if (p.relu_out) v[e] = fmaxf(v[e], 0.f);
            }
            const V2 a0 = cvt2<T>(v[0], v[1]), a1 = cvt2<T>(v[2], v[3]);
            *reinterpret_cast<V4*>(Ow + ln * kDwOss + 8 * q + 4 * g) = V4{a0[0], a0[1], a1[0], a1[1]};
          }
          // 32 channels x 4 vectors of 8 pixels, 64 per pass
#pragma unroll
          for (int v0 = 0; v0 < 128; v0 += 64) {
            const int v = v0 + lane;
            const int ch = v >> 2, sv = v & 3;
            const int c2 = 32 * t + ch;
            const int ph = ov_ph[j], pw = ov_pw[j];
            const V8 px = *reinterpret_cast<const V8*>(Ow + ch * kDwOss + 8 * sv);
            if (c2 < p.C2 && p0 + ph < p.P && q0 + pw < p.Q) {
              V8* dst = reinterpret_cast<V8*>(reinterpret_cast<T*>(p.y) + ((long long)n * p.C2 + c2) * plane +
                                              (long long)(p0 + ph) * p.Q + q0 + pw);
              // streaming stores only where a tile row fills whole 128-byte lines; shorter runs
              // are left to L2 to merge with the neighbouring tile's
              if (p.nt_store) __builtin_nontemporal_store(px, dst);
              else *dst = px;
            }
          }
        }
    } else {
      // o[t][j][r] = out^T[c2 = 32t + 8(r/4) + 4g + r%4][pixel of lane]
#pragma unroll
      for (int t = 0; t < C2T; ++t)
#pragma unroll
        for (int j = 0; j < PXW; ++j) {
          if (sph[j] < 0 || p0 + sph[j] >= p.P || q0 + spw[j] >= p.Q) continue;
          const long long opix = (long long)(p0 + sph[j]) * p.Q + q0 + spw[j];
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int c2 = 32 * t + 8 * (r >> 2) + 4 * g + (r & 3);
            if (c2 >= p.C2) continue;
            float v = o[t][j][r];
            if (p.relu_out) v = fmaxf(v, 0.f);
            const long long off = ((long long)n * p.C2 + c2) * plane + opix;
            if (p.out_f32)
              reinterpret_cast<float*>(p.y)[off] = v;
            else
              reinterpret_cast<T*>(p.y)[off] = (T)v;
          }
        }
    }
  }
#else
  (void)p;
#endif
}

// dwv: depthwise stage on the vector ALU (multipliers 1, 2, 4, 8; 3x3 filters; even cols_al; 16-byte stores)
template <typename T, int C2T, int PXW, int NG>
hipError_t launch_dw_conv_mfma(const DwConvArgs& args, int grid, bool dwv, hipStream_t stream) {
  const bool wide = args.wide != 0;
  const bool f33 = args.R == 3 && args.S == 3 && args.cols_al % 2 == 0;
  if (dwv && !(f33 && wide)) return hipErrorInvalidValue;
  const int lds = dw_conv_mfma_lds_bytes(args.chx, args.mult, args.rows_in, args.cols_al, 32 * C2T, NG, wide);
  void (*kern)(DwConvArgs) = nullptr;
  int slot = 0;
  if (dwv) {
    slot = 4 + (args.mult == 1 ? 0 : args.mult == 2 ? 1 : args.mult == 4 ? 2 : 3);
    kern = args.mult == 1   ? dw_conv_mfma_kernel<T, C2T, PXW, NG, true, true, 0>
           : args.mult == 2 ? dw_conv_mfma_kernel<T, C2T, PXW, NG, true, true, 1>
           : args.mult == 4 ? dw_conv_mfma_kernel<T, C2T, PXW, NG, true, true, 2>
                            : dw_conv_mfma_kernel<T, C2T, PXW, NG, true, true, 3>;
  } else {
    slot = 2 * wide + f33;
    kern = wide ? (f33 ? dw_conv_mfma_kernel<T, C2T, PXW, NG, true, true> : dw_conv_mfma_kernel<T, C2T, PXW, NG, true, false>)
                : (f33 ? dw_conv_mfma_kernel<T, C2T, PXW, NG, false, true> : dw_conv_mfma_kernel<T, C2T, PXW, NG, false, false>);
  }
  static thread_local int configured_dev[8] = {-1, -1, -1, -1, -1, -1, -1, -1};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev[slot] != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev[slot] = dev;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(256 * NG), lds, stream, args);
  return hipGetLastError();
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
