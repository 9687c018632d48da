// Persistent form of the conv(RxS) -> cast|relu -> conv(1x1) chain (conv_chain.h) for chains whose
// weights fit in LDS beside one halo tile.
//
// Reference chain: benchmark/chimera/cuda/conv3x3_conv1x1_cuda.py:77-172.
//
// conv_chain_kernel gives every output tile a workgroup of its own: stage weights and halo tile,
// first convolution, second convolution, stores -- one latency chain per tile, and with about as
// many tiles as the chip holds workgroups all of them run their phases in lockstep, so the output
// (most of the bytes) leaves in the last third of the kernel while HBM idles before.  Here one
// workgroup per CU (eight waves, two per SIMD) keeps both weight tensors for its whole life -- W1 in
// LDS as [tap][c1][C0 + 8], W2 as MFMA operand fragments in registers -- and walks over output tiles
// of full image rows (at most 128 pixels = four MFMA pixel tiles):
//     write the prefetched halo tile to LDS | barrier | issue the loads of the next tile |
//     first convolution, with the second convolution of the PREVIOUS tile dealt out between its
//     steps | exchange | cast | exchange
// Waves w and w + 4 share pixel tile w: each runs half of the first convolution's k steps (taps x
// channel groups), the upper wave hands its partial sums to the lower one through LDS, which adds,
// casts and hands the 16-bit intermediate back; each then computes half of the output channels
// (its half of W2 is 64 registers).  One wave per SIMD was tried first: with nothing to overlap
// them, LDS reads, MFMAs and the output path simply added up (29 us against 14 us with everything
// but the LDS reads removed).
// The second convolution is computed pixel-major; a half-wave swap (v_permlane32_swap) leaves every
// lane with 8 consecutive pixels of one output channel, stored as 16 bytes straight from registers,
// so it touches LDS not at all (measured: with W2 fragments and an output turn-around in LDS the
// kernel was LDS-bandwidth bound at twice the time).
// The stores of tile t are still in flight while tile t+1 is computed: loads and stores go through
// buffer resources (out-of-range lanes are dropped / read zeros by the range check instead of being
// branched around), so their number per tile is fixed and the wait for the next halo tile's loads,
// which are older than the tile's stores, leaves exactly that many operations outstanding.
#pragma once
#include "conv_chain.h"

namespace ditto {


// ReLU on two packed fp16 / bf16 values: as signed 16-bit integers the negative floats (and -0) are
// the negative numbers, so max(x, 0) clears exactly those; with lo = 0x80008000 the max changes
// nothing.  One instruction per two values, the same for both element types, and the rounding that
// came before commutes with it (it keeps sign and zero).
typedef short conv_s16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned conv_relu_pk(unsigned x, unsigned lo) {
  return __builtin_bit_cast(unsigned, __builtin_elementwise_max(__builtin_bit_cast(conv_s16x2, x), __builtin_bit_cast(conv_s16x2, lo)));
}

// f(integral_constant<int, I>) for I = 0 .. N-1: an unrolled loop whose index is a compile-time
// constant in the body (a `#pragma unroll` loop this long is not always unrolled, and then the
// fragment arrays it indexes end up in scratch memory)
template <int I, int N, typename F>
__device__ __forceinline__ void conv_static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>());
    conv_static_for<I + 1, N>(f);
  }
}

__host__ __device__ inline int conv_persist_w1_lds_bytes(int RS, int C1p, int ch) {
  return (conv_w1_chunk_bytes(RS, C1p, ch) + 1023) / 1024 * 1024;  // whole 1 KB direct-load instructions
}
__host__ __device__ inline int conv_persist_x_elems(int rows_in, int cols_in, int ch) {
  return (rows_in * cols_in * conv_ch_stride(ch) + 7) & ~7;
}
// bytes of the exchange buffer: per pixel tile the upper wave's partial sums, C1T x 16 floats per lane
__host__ __device__ inline int conv_persist_xchg_bytes(int C1p) { return 4 * (C1p / 32) * 16 * 64 * 4; }
// halo tile + exchange buffer, or (in the prologue) all 256 rows of W2 at a stride of C1p + 4 elements
__host__ __device__ inline int conv_persist_lds_bytes(int rows_in, int cols_in, int RS, int C1p, int ch) {
  const int work = conv_persist_x_elems(rows_in, cols_in, ch) * 2 + conv_persist_xchg_bytes(C1p);
  const int w2 = 256 * (C1p + 4) * 2;
  return conv_persist_w1_lds_bytes(RS, C1p, ch) + (work > w2 ? work : w2);
}

// Requirements (checked by the host): TW == Q (tiles are runs of whole output rows), TH * TW <= 128,
// Q and W multiples of 8, x / y / w2 16-byte aligned, input and 16-bit output of fewer than 2^31 bytes each, the repacked
// W1 (one chunk of CH channels) in p.w1p, C0 <= CH, C1 <= 32 * C1T, C2 <= 32 * C2T, a square first filter
// R = S = RF, at most one staging task per thread (512), and the LDS footprint above within 160 KB.
template <typename T, int C1T, int CH, int C2T, int RF>
__global__ __launch_bounds__(512) void conv_chain_persist_kernel(ConvChainArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  constexpr int C1p = 32 * C1T;
  constexpr int CHS = conv_ch_stride(CH);
  constexpr int NTH = 512;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  const int RS = p.R * p.S;
  const int w1_bytes = conv_w1_chunk_bytes(RS, C1p, CH);
  const int w1_lds = conv_persist_w1_lds_bytes(RS, C1p, CH);
  const int xs_elems = conv_persist_x_elems(p.rows_in, p.cols_in, CH);
  T* const W1s = reinterpret_cast<T*>(smem_raw);            // [R*S][C1p][CHS]
  T* const Xs = reinterpret_cast<T*>(smem_raw + w1_lds);    // [rows_in][cols_in][CHS]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int pt = wave & 3, kh = wave >> 2;  // pixel tile; half of the k steps / of the output channels
  const int ln = lane & 31, g = lane >> 5;
  // exchange buffer of this pixel tile: 16 bytes per lane and quad of accumulator registers
  // (the intermediate fragments later overlay its start)
  char* const Xc = smem_raw + w1_lds + xs_elems * 2 + pt * (C1T * 4 * 1024) + lane * 16;

  const int ntiles = p.N * p.tiles_h;
  const int plane = p.P * p.Q;
  const T* __restrict__ W2g = reinterpret_cast<const T*>(p.w2);

  // ---- weights, once: W1 (repacked) by direct loads
  {
    const i32x4 w1_rsrc = make_rsrc(p.w1p, (unsigned)w1_bytes);
    const unsigned w1_base = (unsigned)(size_t)(DITTO_LDS char*)smem_raw;
    for (int j = wave; j * 1024 < w1_bytes; j += 8) {
      const int off = j * 1024 + lane * 16;
      lds_dma_16(w1_rsrc, off < w1_bytes ? (unsigned)off : 0x7fffffffu, w1_base + j * 1024);
    }
  }
  // This wave's half of W2 as operand fragments, in registers for the whole kernel: for k step u of its
  // output-channel block b (channels 32 (NB kh + b) ..) the lane holds W2[c2 = .. + ln][16u + 4g + {0..3}]
  // and [16u + 8 + 4g + {0..3}] (zero past C2 / C1).  W2 passes through LDS (the halo tile and exchange
  // areas, not yet in use) with 16-byte loads: fetched straight from memory the fragments are 8-byte
  // pieces of 32 different rows per load, an L2 request each (5.7 us of a 9 us prologue measured).
  static_assert(C2T % 2 == 0 && 32 * C2T <= 256, "the output channel blocks are split between two waves; the LDS size allows for 256 rows of W2");
  constexpr int NB = C2T / 2;
  constexpr int W2S = C1p + 4;  // row stride (elements): conflict-free 8-byte reads
  V8 w2r[NB][2 * C1T];
  {
    T* const W2s = Xs;
    constexpr int VPR = C1p / 8;  // 16-byte vectors per row
    for (int e = tid; e < 32 * C2T * VPR; e += NTH) {
      const int row = e / VPR, vc = e % VPR;
      i32x4 v = {0, 0, 0, 0};
      if (row < p.C2 && 8 * vc < p.C1) v = *reinterpret_cast<const i32x4*>(W2g + (long long)row * p.C1 + 8 * vc);
      *reinterpret_cast<i32x2*>(W2s + row * W2S + 8 * vc) = i32x2{v[0], v[1]};  // rows are only 8-byte aligned
      *reinterpret_cast<i32x2*>(W2s + row * W2S + 8 * vc + 4) = i32x2{v[2], v[3]};
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
      for (int u = 0; u < 2 * C1T; ++u) {
        const T* wr = W2s + (32 * (NB * kh + b) + ln) * W2S + 16 * u + 4 * g;
        w2r[b][u] = concat4<V4, V8>(*reinterpret_cast<const V4*>(wr), *reinterpret_cast<const V4*>(wr + 8));
      }
    __syncthreads();  // before the area is zeroed below
  }
  // the halo tile's padding columns are never written again: zero the whole tile once
  for (int e = tid; e * 8 < xs_elems; e += NTH) *reinterpret_cast<i32x4*>(Xs + 8 * e) = i32x4{0, 0, 0, 0};

  // ---- pixel slot of this lane (the same in every tile): slot = 32 * pt + ln -> (ph, pw)
  const int slot_l = 32 * pt + ln;
  const int ph_l = slot_l / p.TW, pw_l = slot_l - ph_l * p.TW;
  const int xoff = ph_l < p.TH ? ((ph_l * p.stride) * p.cols_in + pw_l * p.stride) * CHS + 8 * g : 8 * g;

  // ---- halo staging: a task is an aligned group of 8 pixels x 8 channels of one halo row inside
  // the image: eight 16-byte loads (one per channel), an 8x8 transposition in registers, eight
  // 16-byte LDS writes (one per pixel).  Columns left and right of the image stay zero.
  const int ngc = p.W >> 3;
  const int xtasks = p.rows_in * ngc * (CH / 8);
  i32x4 xr[8];
  const int t_chg = tid % (CH / 8), t_gi = (tid / (CH / 8)) % ngc, t_ri = tid / (CH / 8) / ngc;
  // Range-checked buffer loads: a task outside the image or past C0 reads zeros from an offset beyond
  // the tensor, so the number of loads per tile is fixed.  They are issued as inline asm, which keeps
  // them out of the compiler's own wait-count bookkeeping (it would wait for everything outstanding,
  // the previous tile's stores included, before the first use): xv_wait() below is the wait.
  // INVARIANT: until that wait nothing may read, copy or spill the destination registers (a copy
  // made by the register allocator would take stale values and free a register that the returning
  // load then overwrites); tests/test_async_registers.py checks the generated code for it.
  const i32x4 x_rsrc = make_rsrc(p.x, (unsigned)(p.N * p.C0 * p.H * p.W * 2));
  const int hw2 = p.H * p.W * 2;  // bytes of one channel plane
  auto xv_load = [&](int tile) __attribute__((always_inline)) {
    const int n = tile / p.tiles_h, th = tile - n * p.tiles_h;
    const int h = th * p.TH * p.stride - p.pad + t_ri;
    const bool ok = tid < xtasks && h >= 0 && h < p.H;
    const int base = ((n * p.C0 + 8 * t_chg) * p.H + h) * p.W * 2 + 16 * t_gi;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      // (no short-circuit: the loads must stay straight-line code)
      const unsigned in = (unsigned)ok & (unsigned)(8 * t_chg + c < p.C0);
      const unsigned off = in ? (unsigned)(base + c * hw2) : 0x7ffffff0u;
      asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(xr[c]) : "v"(off), "s"(x_rsrc) : "memory");
    }
  };
  // Wait until at most `newer` vector-memory operations issued after the last xv_load are outstanding
  // (they complete in order): `newer` = the stores of one tile.  The halo registers are operands so that
  // no use of them can be scheduled above the wait.
  constexpr int NEWER = C2T;  // 2 stores for each of the wave's C2T / 2 output-channel blocks
  auto xv_wait = [&]() __attribute__((always_inline)) {
    asm volatile("s_waitcnt vmcnt(%8)"
                 : "+v"(xr[0]), "+v"(xr[1]), "+v"(xr[2]), "+v"(xr[3]), "+v"(xr[4]), "+v"(xr[5]), "+v"(xr[6]), "+v"(xr[7])
                 : "n"(NEWER));
  };
  auto xv_store = [&]() __attribute__((always_inline)) {
    const int ci0 = 8 * t_gi + p.pad;  // halo column of the group's first pixel
#pragma unroll
    for (int px = 0; px < 8; ++px) {
      i32x4 o;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        o[d] = __builtin_amdgcn_perm(xr[2 * d + 1][px >> 1], xr[2 * d][px >> 1], (px & 1) ? 0x07060302 : 0x05040100);
      const int ci = ci0 + px;
      if (tid < xtasks && ci < p.cols_in) *reinterpret_cast<i32x4*>(Xs + (t_ri * p.cols_in + ci) * CHS + 8 * t_chg) = o;
    }
  };

  // ---- output through a range-checked buffer resource (dropped stores keep the count per tile fixed)
  const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.y, 0, p.N * p.C2 * plane * 2, 0x00020000);

  // ---- second convolution (1x1) of one tile, operands swapped: o[r] = out[pixel 8(r/4) + 4g + r%4][c2 =
  // 32 (NB kh + b) + ln], one block of 32 output channels at a time.  The state of the tile it works on
  // (cast intermediate, output offset, valid pixels) is carried from the previous pass of the tile
  // loop: its blocks are spread over the first convolution of the next tile so that the output leaves
  // at an even rate instead of in a burst after every tile.
  V8 pf[2 * C1T];
#pragma unroll
  for (int u = 0; u < 2 * C1T; ++u) pf[u] = V8{0, 0, 0, 0, 0, 0, 0, 0};
  int img_off = 0, nvalid = 0;  // no valid pixel: before the first tile the stores are all dropped
  const unsigned relu_mid_lo = p.relu_mid ? 0u : 0x80008000u, relu_out_lo = p.relu_out ? 0u : 0x80008000u;
  f32x16 o2;
  auto st_mfma = [&](int b) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; ++r) o2[r] = 0.f;
#pragma unroll
    for (int u = 0; u < 2 * C1T; ++u) o2 = Elem<T>::mfma32(pf[u], w2r[b][u], o2);
  };
  // Registers 4q .. 4q+3 are pixels 8q + 4g + {0..3} of channel .. + ln.  Swapping the packed quads of
  // q0 = 2j (kept by the lower half-wave) and q1 = 2j + 1 (kept by the upper) between the half-waves
  // gives lane (ln, g) the 8 pixels 8(2j + g) .. +7: one 16-byte store.
  auto st_out = [&](int b) __attribute__((always_inline)) {
    unsigned d[4][2];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      d[q][0] = conv_relu_pk(__builtin_bit_cast(unsigned, cvt2<T>(o2[4 * q + 0], o2[4 * q + 1])), relu_out_lo);
      d[q][1] = conv_relu_pk(__builtin_bit_cast(unsigned, cvt2<T>(o2[4 * q + 2], o2[4 * q + 3])), relu_out_lo);
    }
    const int c2 = 32 * (NB * kh + b) + ln;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const auto s0 = __builtin_amdgcn_permlane32_swap(d[2 * j][0], d[2 * j + 1][0], false, false);
      const auto s1 = __builtin_amdgcn_permlane32_swap(d[2 * j][1], d[2 * j + 1][1], false, false);
      const u32x4 px = {s0[0], s1[0], s0[1], s1[1]};
      const int slot = 32 * pt + 8 * (2 * j + g);
      const bool ok = c2 < p.C2 && slot < nvalid;
      const unsigned off = ok ? (unsigned)(img_off + (c2 * plane + slot) * 2) : 0x7ffffff0u;
      __builtin_amdgcn_raw_buffer_store_b128(px, y_rsrc, off, 0, 0);
    }
  };

  // ---- this wave's half of the first convolution (k steps K0 .. K0 + KH - 1), unrolled; the operand
  // fragments of step k + kAhead are fetched before the MFMAs of step k and the scheduling barriers
  // keep the compiler from collapsing that distance.  Long halves (STAGED): block b of the previous
  // tile's second convolution has its MFMAs behind those of step b * SPB and its conversion and stores
  // before the MFMAs of step b * SPB + 2; short ones: all blocks after the last step.
  f32x16 acc[C1T];
  constexpr int KK = CH / 16, K = RF * RF * KK, KH = K / 2;
  static_assert(K % 2 == 0, "the k steps are split between two waves");
  constexpr int SPB = KH / NB;
  constexpr bool STAGED = SPB >= 3 && (NB - 1) * SPB + 2 <= KH - 1;
  auto conv1_half = [&](auto k0_c) __attribute__((always_inline)) {
    constexpr int K0 = decltype(k0_c)::value;
    constexpr int kAhead = 4;
    const T* xl = Xs + xoff;
    const T* wl = W1s + ln * CHS + 8 * g;
    V8 xf[KH], wf[KH][C1T];
    auto ld = [&](int kl) __attribute__((always_inline)) {
      const int k = K0 + kl, tap = k / KK, kk = k % KK;
      xf[kl] = *reinterpret_cast<const V8*>(xl + ((tap / RF) * p.cols_in + tap % RF) * CHS + 16 * kk);
#pragma unroll
      for (int c = 0; c < C1T; ++c) wf[kl][c] = *reinterpret_cast<const V8*>(wl + (tap * C1p + 32 * c) * CHS + 16 * kk);
    };
#pragma unroll
    for (int kl = 0; kl < kAhead && kl < KH; ++kl) ld(kl);
    conv_static_for<0, KH>([&](auto kc) __attribute__((always_inline)) {
      constexpr int kl = decltype(kc)::value;
      if (kl + kAhead < KH) ld(kl + kAhead);
      if constexpr (STAGED) {
        if (kl >= 2 && (kl - 2) % SPB == 0 && (kl - 2) / SPB < NB) st_out((kl - 2) / SPB);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int c = 0; c < C1T; ++c) acc[c] = Elem<T>::mfma32(wf[kl][c], xf[kl], acc[c]);
      if constexpr (STAGED) {
        if (kl % SPB == 0 && kl / SPB < NB) st_mfma(kl / SPB);
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
  int tile = (int)lid;
  if (tile < ntiles) xv_load(tile);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the direct loads of W1 (and the first halo tile) have landed
  __syncthreads();  // ... in every wave; the zero fill is ordered before the first halo writes
  while (tile < ntiles) {
    const int next = tile + (int)gridDim.x;
    // every pass issues the 2 * NB stores of the previous tile (dropped ones before the first) after
    // the loads of the next halo tile: that many operations may stay in flight here
    xv_wait();
    xv_store();
    __syncthreads();
    if (next < ntiles) xv_load(next);  // in flight during the MFMAs

#pragma unroll
    for (int c = 0; c < C1T; ++c)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
    if (kh == 0) conv1_half(std::integral_constant<int, 0>());
    else conv1_half(std::integral_constant<int, KH>());
    if constexpr (!STAGED) {
#pragma unroll
      for (int b = 0; b < NB; ++b) {
        st_mfma(b);
        st_out(b);
      }
    }

    // ---- the upper wave's partial sums go to the lower one, which adds, applies the inter op and
    // casts: mid^T tile c regs 8(u%2)..+7 are the operand of k step u of the second convolution
    // (channels 16u + 4g + {0..3} and 16u + 8 + 4g + {0..3}); the fragments go back the same way
    if (kh == 1) {
#pragma unroll
      for (int c = 0; c < C1T; ++c)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          *reinterpret_cast<f32x4*>(Xc + (4 * c + q) * 1024) = f32x4{acc[c][4 * q], acc[c][4 * q + 1], acc[c][4 * q + 2], acc[c][4 * q + 3]};
    }
    __syncthreads();  // partial sums visible; every wave is done with the halo tile
    if (kh == 0) {
#pragma unroll
      for (int c = 0; c < C1T; ++c)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4 o = *reinterpret_cast<const f32x4*>(Xc + (4 * c + q) * 1024);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[c][4 * q + e] += o[e];
        }
#pragma unroll
      for (int c = 0; c < C1T; ++c)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          u32x4 w;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            w[e] = conv_relu_pk(__builtin_bit_cast(unsigned, cvt2<T>(acc[c][8 * hh + 2 * e], acc[c][8 * hh + 2 * e + 1])), relu_mid_lo);
          pf[2 * c + hh] = __builtin_bit_cast(V8, w);
          *reinterpret_cast<u32x4*>(Xc + (2 * c + hh) * 1024) = w;  // over the sums read above (this wave's own)
        }
    }
    __syncthreads();
    if (kh == 1) {
#pragma unroll
      for (int u = 0; u < 2 * C1T; ++u) pf[u] = *reinterpret_cast<const V8*>(Xc + u * 1024);
    }
    {
      const int n = tile / p.tiles_h, th = tile - n * p.tiles_h;
      const int p0 = th * p.TH;
      nvalid = (p.P - p0 < p.TH ? p.P - p0 : p.TH) * p.Q;
      img_off = (n * p.C2 * plane + p0 * p.Q) * 2;  // bytes; the whole output is below 2^31 bytes
    }
    tile = next;
  }
  // the last tile's second convolution
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    st_mfma(b);
    st_out(b);
  }
#else
  (void)p;
#endif
}

template <typename T, int C1T, int CH, int C2T, int RF>
hipError_t launch_conv_chain_persist(const ConvChainArgs& args, int grid, hipStream_t stream) {
  const int lds = conv_persist_lds_bytes(args.rows_in, args.cols_in, args.R * args.S, 32 * C1T, CH);
  auto kern = conv_chain_persist_kernel<T, C1T, CH, C2T, RF>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(512), lds, stream, args);
  return hipGetLastError();
}

}  // namespace ditto
