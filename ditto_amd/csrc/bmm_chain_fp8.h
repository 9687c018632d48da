// Eight-wave variant of the fused two-contraction chain (see bmm_chain_fp.h for the chain,
// the transposed formulation and the operand layouts).
//
// A wave of the four-wave kernel issues one instruction stream per SIMD: while an MFMA
// occupies its issue slot nothing else of that wave can issue, so at most two or three VALU
// instructions hide under each MFMA and the softmax (about four per MFMA) does not.  Here a
// workgroup has EIGHT waves, two per SIMD, each owning 32 rows of A with at most 256
// registers: the hardware interleaves the two instruction streams, so one wave's
// exponentials run under the other wave's MFMAs without any software pipelining.
//
// The price is LDS traffic: with 32 rows per wave every operand fragment read from LDS feeds
// a single MFMA.  16-byte row reads sustain that (256 B/clk per CU); the transposing read
// ds_read_b64_tr_b16 moves half as many bytes per instruction (128 B/clk under these tiles' swizzle,
// 220 B/clk at best), so the same fragments cost twice the LDS instructions, and with every wave
// reading its fragments that way the 16x16x32 kernel was 4.5 % slower than with the pass below.
// So every tile whose contraction index is
// the row index (C always, B in [K][L] layout) is transposed ONCE per workgroup: the wave
// that owns a fragment reads it with the transposing read and writes it back "fragment
// major" (1 KB per fragment, lane l at byte 16*l), after which all eight waves fetch it with
// plain, conflict-free 16-byte reads.
//
// Pipeline per L tile `it` (one barrier per tile):
//   direct loads   B(it+2) (row-read layout) or B(it+3) (raw, [K][L] layout), C(it+2) (raw)
//   transposition  raw C(it+1) -> fragment-major C(it+1); raw B(it+2) -> fragment-major B(it+2)
//   compute        waves 0-3: S(it) = B(it)^T.A^T, inter op, F^T += C(it)^T.P(it)^T
//                  waves 4-7: inter op on S(it), F^T += C(it)^T.P(it)^T, S(it+1)
//
// PIPE = true is the software-pipelined form of the compute part.  Above, a wave alternates between
// MFMA-only and vector-only phases and the overlap comes from running the two waves of a SIMD half a
// tile apart; the phases differ in length, so the waves drift and one of them waits at every barrier.
// Pipelined, every wave runs the SAME stream in half steps of 32 rows of the L tile, as the four-wave
// kernel does: while the matrix pipe computes the scores of the next half, the vector ALU
// exponentiates the current one, a few vector instructions behind every MFMA (an MFMA holds the vector
// issue port for about 12 of its 32 cycles, which leaves the two waves of a SIMD five vector issue
// slots per MFMA).  The waves stay level and reach the barrier together.
#pragma once
#include <type_traits>
#include "bmm_chain_fp.h"

namespace ditto {

// Raw C tiles kept in LDS: two (a tile is loaded two steps before its use) or, where LDS allows
// (head_pad 64 with B consumed as loaded), four, so that loads run three steps ahead -- one step
// of a short tile does not cover the memory latency.
template <int D, bool B_KL>
__host__ __device__ constexpr int bmm_chain8_raw_c_tiles() {
  return (D == 64 && !B_KL) ? 4 : 2;
}

template <int D, bool B_KL>
__host__ __device__ constexpr int bmm_chain8_lds_bytes() {
  return ((B_KL ? 6 : 4) + bmm_chain8_raw_c_tiles<D, B_KL>() + 2) * kBN * D * 2;
}

template <typename T, int D, int INTER, bool B_KL, bool PIPE = false>
__global__ __launch_bounds__(512) void bmm_chain8_kernel(BmmChainArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  typedef typename Elem<T>::v2 V2;
  constexpr int NW = 8, BM = NW * 32;
  constexpr int TB = kBN * D * 2;               // bytes per tile
  constexpr int B_RB = B_KL ? kBN * 2 : D * 2;  // bytes per LDS row of a B tile as loaded
  constexpr int B_CPR = B_RB / 16;
  constexpr int C_RB = D * 2;
  constexpr int C_CPR = C_RB / 16;
  constexpr int NS = D / 16;                    // MFMA k steps of the first contraction per 32 rows
  constexpr int NT = D / 32;                    // column tiles of the second contraction
  constexpr int NFRAG = 2 * NS;                 // fragments per tile (B and C alike)
  constexpr int NLD = TB / 1024 / NW;           // direct loads per wave per tile
  constexpr int NTR = NFRAG / NW;               // fragments each wave transposes per tile
  static_assert(NLD >= 1 && NTR >= 1, "tile too small for eight waves");
  // LDS map (bytes): B tiles, then raw C tiles, then fragment-major C tiles
  constexpr int B_LOAD = 0;                             // as loaded: [4] row-read layout, or [2] raw
  constexpr int B_FRAG = 2 * TB;                        // [4] fragment major (B_KL only)
  constexpr int NCR = bmm_chain8_raw_c_tiles<D, B_KL>();
  constexpr int C_RAW = (B_KL ? 6 : 4) * TB;            // [NCR]
  constexpr int C_FRAG = C_RAW + NCR * TB;              // [2]
  // loads run this many steps ahead of the step that consumes them
  constexpr int B_AHEAD = 3;                            // (B_KL: into the raw pair, transposed a step later)
  constexpr int C_AHEAD = NCR == 4 ? 3 : 2;
  constexpr int B_USE = B_KL ? B_FRAG : B_LOAD;         // the four buffers the first contraction reads

  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int i16 = lane & 15, h = (lane >> 4) & 1;
  // The two waves of a SIMD (w and w+4) run half a tile apart: the "late" wave computes the
  // scores of tile it+1 at the END of step it, so its softmax of step it+1 runs while the
  // other wave's MFMAs occupy the matrix pipe, and vice versa.
  const bool late = !PIPE && wave >= 4;

  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
  const int mb = lid % p.mblocks;
  const int bz = lid / p.mblocks;
  // batch entry bz = zo * batch_inner + zi
  const int zo = bz / p.batch_inner, zi = bz - zo * p.batch_inner;
  const T* __restrict__ Ag = reinterpret_cast<const T*>(p.a) + zo * p.a_bs2 + zi * p.a_bs;
  const T* Bg = reinterpret_cast<const T*>(p.b) + zo * p.b_bs2 + zi * p.b_bs;
  const T* Cg = reinterpret_cast<const T*>(p.c) + zo * p.c_bs2 + zi * p.c_bs;
  const int m_wave = mb * BM + wave * 32;
  const int M = p.M, N = p.N, K = p.K, L = p.L;

  const unsigned b_bytes = (unsigned)(B_KL ? ((long long)(K - 1) * p.b_rs + L) : ((long long)(L - 1) * p.b_rs + K)) * 2u;
  const unsigned c_bytes = (unsigned)((long long)(L - 1) * p.c_rs + N) * 2u;
  const i32x4 b_rsrc = make_rsrc(Bg, b_bytes);
  const i32x4 c_rsrc = make_rsrc(Cg, c_bytes);
  const unsigned lds0 = (unsigned)(size_t)(DITTO_LDS char*)smem_raw;

  // ---- per-lane source offsets of the direct loads (same swizzles as the four-wave kernel)
  int b_voff[NLD], c_voff[NLD], b_col[NLD];
#pragma unroll
  for (int q = 0; q < NLD; ++q) {
    const int gi = NLD * wave + q;
    {
      const int row = gi * (64 / B_CPR) + lane / B_CPR, pc = lane % B_CPR;
      if (B_KL) {
        const int cl = pc ^ swz_trread<B_CPR>(row);
        b_col[q] = cl * 8;
        b_voff[q] = row < K ? (row * p.b_rs + cl * 8) * 2 : (int)b_bytes;
      } else {
        const int cl = pc ^ swz_rowread<B_CPR>(row);
        b_col[q] = 0;
        b_voff[q] = cl * 8 < K ? (row * p.b_rs + cl * 8) * 2 : (int)b_bytes;
      }
    }
    {
      const int row = gi * (64 / C_CPR) + lane / C_CPR, pc = lane % C_CPR;
      const int cl = pc ^ swz_trread<C_CPR>(row);
      c_voff[q] = cl * 8 < N ? (row * p.c_rs + cl * 8) * 2 : (int)c_bytes;
    }
  }
  auto load_b = [&](int tile, int buf) __attribute__((always_inline)) {
    const int l0 = tile * kBN;
    const int soff = B_KL ? l0 * 2 : l0 * p.b_rs * 2;
#pragma unroll
    for (int q = 0; q < NLD; ++q) {
      int vo = b_voff[q] + soff;
      if (B_KL) vo = (l0 + b_col[q] < L) ? vo : (int)b_bytes;
      lds_dma_16(b_rsrc, (unsigned)vo, lds0 + B_LOAD + buf * TB + 1024 * (NLD * wave + q));
    }
  };
  auto load_c = [&](int tile, int buf) __attribute__((always_inline)) {
    const int soff = tile * kBN * p.c_rs * 2;
#pragma unroll
    for (int q = 0; q < NLD; ++q)
      lds_dma_16(c_rsrc, (unsigned)(c_voff[q] + soff), lds0 + C_RAW + buf * TB + 1024 * (NLD * wave + q));
  };

  // ---- per-lane LDS read addresses (bytes within a tile), loop invariant
  const int b_rd = B_KL ? ((8 * g + (i16 >> 2)) * B_RB + (2 * h + ((i16 & 3) >> 1)) * 16 + 8 * (i16 & 1))
                        : (ln * B_RB);
  const int c_rd = (4 * g + (i16 >> 2)) * C_RB + (2 * h + ((i16 & 3) >> 1)) * 16 + 8 * (i16 & 1);
  int b_ad[2][NS], c_ad[NT];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int x = B_KL ? swz_trread<B_CPR>(i16 >> 2) : (g ^ swz_rowread<B_CPR>(32 * i + ln));
#pragma unroll
    for (int st = 0; st < NS; ++st) b_ad[i][st] = b_rd + (B_KL ? ((4 * i) ^ x) : ((2 * st) ^ x)) * 16;
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) c_ad[t] = c_rd + ((4 * t) ^ swz_trread<C_CPR>(i16 >> 2)) * 16;
  const int frag_ad = lane * 16;

  // a row-read B fragment (plain 16-byte read) and a fragment-major fragment
  auto b_frag_row = [&](int off, int i, int st) __attribute__((always_inline)) -> V8 {
    return *reinterpret_cast<const V8*>(smem_raw + b_ad[i][st] + (off + 32 * i * B_RB));
  };
  auto frag_rd = [&](int off, int f) __attribute__((always_inline)) -> V8 {
    return *reinterpret_cast<const V8*>(smem_raw + frag_ad + (off + 1024 * f));
  };
  // This wave's share of the transposition of one tile: fragments NTR*wave .. +NTR-1
  // (C fragment f = u*NT + t: rows 16u.., columns 32t..; B fragment f = i*NS + st: rows 16st..,
  // columns 32i..).  The per-lane source addresses are wave dependent, computed once.
  int ctr_ad[NTR], btr_ad[NTR], fw_ad[NTR];
#pragma unroll
  for (int q = 0; q < NTR; ++q) {
    const int f = NTR * wave + q;
    ctr_ad[q] = c_rd + ((4 * (f % NT)) ^ swz_trread<C_CPR>(i16 >> 2)) * 16 + 16 * (f / NT) * C_RB;
    btr_ad[q] = B_KL ? b_rd + ((4 * (f / NS)) ^ swz_trread<B_CPR>(i16 >> 2)) * 16 + 16 * (f % NS) * B_RB : 0;
    fw_ad[q] = frag_ad + 1024 * f;
  }
  auto tr_read_c = [&](int raw_off, V8* x) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < NTR; ++q) {
      const char* a = smem_raw + ctr_ad[q] + raw_off;
      V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(a));
      V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(a + 8 * C_RB));
      x[q] = concat4<V4, V8>(lo, hi);
    }
  };
  auto tr_read_b = [&](int raw_off, V8* x) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < NTR; ++q) {
      const char* a = smem_raw + btr_ad[q] + raw_off;
      V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(a));
      V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(a + 4 * B_RB));
      x[q] = concat4<V4, V8>(lo, hi);
    }
  };
  auto tr_write = [&](int frag_off, const V8* x) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < NTR; ++q) *reinterpret_cast<V8*>(smem_raw + fw_ad[q] + frag_off) = x[q];
  };

  // ---- A fragments (B operand of D^T = B^T.A^T): lane holds A[row][16s + 8g .. +7]
  V8 af[NS];
  {
    const int row = m_wave + ln;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int col = 16 * s + 8 * g;
      V8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (row < M && col < K) v = *reinterpret_cast<const V8*>(Ag + (long long)row * p.a_rs + col);
      af[s] = v;
    }
  }
  // Pre-scaled softmax (fp16, pipelined kernel): A is multiplied by scale * log2(e) ONCE, here, and the first MFMA
  // of every score tile starts from minus the row's running maximum instead of zero, so the accumulator already
  // holds the exponent: a score then costs its v_exp_f32 and nothing else (the multiply-add in front of it was a
  // sixth of the vector work that bounds this kernel at head dimension 64: 13.9 -> 12.7 us per call on
  // 96 x 512 x 64).  The price is one more fp16 rounding of A (2^-11 relative: rel-L2 of the result
  // 2.9e-4 -> 3.5e-4 at 4096 x 128); bf16 would pay 2^-9 there (2.3e-3 -> 2.9e-3) and stays on the exact form.
  // (head dimension 64 only: at 128 the sixteen more registers do not fit without scratch)
  constexpr bool PRE = PIPE && INTER == kInterSoftmax && std::is_same<T, f16>::value && D <= 64;
  if constexpr (PRE) {
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const V2 q2 = cvt2<T>((float)af[s][e] * p.scale_log2, (float)af[s][e + 1] * p.scale_log2);
        af[s][e] = q2[0];
        af[s][e + 1] = q2[1];
      }
  }

  // ---- accumulators of F^T: o[t][r] = F^T[32t + 8(r/4) + 4g + r%4][ln]
  f32x16 o[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[t][r] = 0.f;
  // (pre-scaled form: scores are kept relative to the running maximum, which starts at zero and is set from the
  // first half tile; negm = sixteen copies of minus that maximum, the accumulator a score tile starts from)
  float mrow = PRE ? 0.f : -INFINITY, lsum = 0.f;
  f32x16 negm = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  const float c2 = p.scale_log2;
  const int ntiles = (L + kBN - 1) / kBN;
  const bool ragged = (L % kBN) != 0;

  // Operand fragments are fetched kAhead MFMAs ahead of their use; the scheduling barriers keep
  // the compiler from collapsing the prefetch distance (it otherwise reuses one register set
  // and waits for every fragment).
  constexpr int kAhead = 4;
  f32x16 s[2];
  // first contraction, transposed: s[i] = (B^T rows 32i..32i+31) . A^T; MFMA k = 2*st + i
  auto scores = [&](auto off_c) __attribute__((always_inline)) {
    constexpr int OFF = decltype(off_c)::value;
    auto rd = [&](int k) __attribute__((always_inline)) -> V8 {
      return B_KL ? frag_rd(OFF, (k & 1) * NS + (k >> 1)) : b_frag_row(OFF, k & 1, k >> 1);
    };
    V8 fr[2 * NS];
#pragma unroll
    for (int k = 0; k < kAhead; ++k) fr[k] = rd(k);
#pragma unroll
    for (int k = 0; k < 2 * NS; ++k) {
      if (k + kAhead < 2 * NS) fr[k + kAhead] = rd(k + kAhead);
      __builtin_amdgcn_sched_barrier(0);
      if (k < 2) {
        const f32x16 z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        s[k & 1] = Elem<T>::mfma32(fr[k], af[k >> 1], z);
      } else {
        s[k & 1] = Elem<T>::mfma32(fr[k], af[k >> 1], s[k & 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // One L tile.  J = it % 4 selects the buffers of tile it (compile time).
  auto tile_step = [&](int it, auto j_c) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;
    constexpr int PAR = J & 1;
    constexpr int CF = C_FRAG + PAR * TB;
    // loads ahead (tiles past the end are out of range and load zeros); transposition reads
    V8 xb[NTR], xc[NTR];
    // C first: the wait at the end of the step can then leave the (younger) B loads in flight
    load_c(it + C_AHEAD, NCR == 4 ? (J + 3) % 4 : PAR);
    load_b(it + B_AHEAD, B_KL ? (PAR ^ 1) : (J + 3) % 4);  // not B_KL: the buffer tile it - 1 used
    if (B_KL) tr_read_b(B_LOAD + PAR * TB, xb);
    tr_read_c(C_RAW + (NCR == 4 ? (J + 1) % 4 : (PAR ^ 1)) * TB, xc);

    if (!late) scores(IntC<B_USE + J * TB>{});

    // transposition writes; first fragments of the second contraction
    if (B_KL) tr_write(B_FRAG + ((J + 2) % 4) * TB, xb);
    tr_write(C_FRAG + (PAR ^ 1) * TB, xc);
    V8 fr[4 * NT];
#pragma unroll
    for (int k = 0; k < kAhead; ++k) fr[k] = frag_rd(CF, k);
    __builtin_amdgcn_sched_barrier(0);

    if constexpr (INTER == kInterSoftmax) {
      if (ragged && it == ntiles - 1) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int l = it * kBN + 32 * i + 8 * (r >> 2) + 4 * g + (r & 3);
            s[i][r] = neg_inf_where(s[i][r], (L - 1 - l) >> 31);  // l >= L
          }
      }
      float mx = s[0][0];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[i][r]);
      mx = pair_max(mx) * c2;
      // lazy rescale: raise the running maximum only when a row of the wave exceeds it by 2^kLazy
      if (__builtin_amdgcn_ballot_w64(mx > mrow + kLazy) != 0) {
        const float mnew = fmaxf(mrow, mx);
        const float alpha = __builtin_amdgcn_exp2f(mrow - mnew);
        mrow = mnew;
        lsum *= alpha;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[i][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i][r], c2, -mrow));
    }
    __builtin_amdgcn_sched_barrier(0);

    // second contraction: o[t] += (C^T tile t, rows 16u..16u+15) . (P^T); half-wave g supplies
    // rows 16u + 4g + {0..3} and 16u + 8 + 4g + {0..3}: registers 8(u%2)..+7 of s[u/2].
    // MFMA k = u*NT + t.
    V8 pf;
#pragma unroll
    for (int k = 0; k < 4 * NT; ++k) {
      const int u = k / NT, t = k % NT;
      if (k + kAhead < 4 * NT) fr[k + kAhead] = frag_rd(CF, k + kAhead);
      if (t == 0) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[e] = s[u >> 1][8 * (u & 1) + e];
          if (INTER != kInterSoftmax && p.relu) v[e] = fmaxf(v[e], 0.f);
        }
        V2 p0 = cvt2<T>(v[0], v[1]), p1 = cvt2<T>(v[2], v[3]), p2 = cvt2<T>(v[4], v[5]), p3 = cvt2<T>(v[6], v[7]);
        if constexpr (INTER == kInterSoftmax) {
          // row sum over the ROUNDED probabilities: exactly what enters the MFMA
          lsum = Elem<T>::add_pair(p0, lsum);
          lsum = Elem<T>::add_pair(p1, lsum);
          lsum = Elem<T>::add_pair(p2, lsum);
          lsum = Elem<T>::add_pair(p3, lsum);
        }
        pf = V8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
      }
      __builtin_amdgcn_sched_barrier(0);
      o[t] = Elem<T>::mfma32(fr[k], pf, o[t]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (late && it + 1 < ntiles) scores(IntC<B_USE + ((J + 1) % 4) * TB>{});
    // everything the next step reads has landed; what this step issued may stay in flight: its B
    // loads always (B as loaded is consumed two steps on at the earliest), its C loads when there
    // are four raw C tiles
    if (B_KL) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (NCR == 4) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NLD) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLD) : "memory");
    __syncthreads();
  };


  // ======== pipelined form (PIPE) ========
  // sa / sb alternate as the finished half (`cur`) and the half being computed (`nxt`); mxn is the scaled
  // row maximum of `cur`.
  f32x16 sa, sb;
  float mxn = -INFINITY;
  auto b_frag = [&](int off, int i, int st) __attribute__((always_inline)) -> V8 {
    return B_KL ? frag_rd(off, i * NS + st) : b_frag_row(off, i, st);
  };
  // scores of rows past L are masked out (softmax only; the other chains see zero operands)
  auto mask_tail = [&](f32x16& sc, int l0) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int l = l0 + 8 * (r >> 2) + 4 * g + (r & 3);
      sc[r] = neg_inf_where(sc[r], (L - 1 - l) >> 31);  // l >= L
    }
  };
  auto row_max = [&](const f32x16& sc) __attribute__((always_inline)) {
    float mx = sc[0];
#pragma unroll
    for (int r = 1; r < 16; ++r) mx = fmaxf(mx, sc[r]);
    mxn = PRE ? pair_max(mx) : pair_max(mx) * c2;  // (pre-scaled: already an exponent, relative to mrow)
  };
  // probabilities of registers [r0, r1) of the half tile
  auto exp_range = [&](f32x16& sc, int r0, int r1) __attribute__((always_inline)) {
#pragma unroll
    for (int r = r0; r < r1; ++r)
      sc[r] = PRE ? __builtin_amdgcn_exp2f(sc[r]) : __builtin_amdgcn_exp2f(__builtin_fmaf(sc[r], c2, -mrow));
  };
  // operand of the second contraction for sixteen rows of the L tile: registers 8 * u2 .. + 7 of the half,
  // cast; the row sum is taken over the ROUNDED values, exactly what enters the MFMA
  auto make_p = [&](const f32x16& sc, int u2, V8& pf) __attribute__((always_inline)) {
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[e] = sc[8 * u2 + e];
      if (INTER != kInterSoftmax && p.relu) v[e] = fmaxf(v[e], 0.f);
    }
    V2 p0 = cvt2<T>(v[0], v[1]), p1 = cvt2<T>(v[2], v[3]), p2 = cvt2<T>(v[4], v[5]), p3 = cvt2<T>(v[6], v[7]);
    if constexpr (INTER == kInterSoftmax) {
      lsum = Elem<T>::add_pair(p0, lsum);
      lsum = Elem<T>::add_pair(p1, lsum);
      lsum = Elem<T>::add_pair(p2, lsum);
      lsum = Elem<T>::add_pair(p3, lsum);
    }
    pf = V8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  };
  // One half step: consumes `cur` (half hh of tile it) and produces `nxt` (half 1 of the same tile, or
  // half 0 of tile it + 1; past the last tile that is a tile of zeros whose scores nothing reads).
  // NS MFMAs of the first contraction, then two sixteen-row steps x NT column tiles of the second.
  // Of the sixteen exponentials per lane EA run behind the first contraction's MFMAs (at least the eight
  // that the first sixteen-row step needs), the rest behind the first NT MFMAs of the second.
  constexpr int NG = NS + 2 * NT;
  constexpr int EA = D == 128 ? 12 : 10;
  static_assert(EA >= 8 && EA <= 16, "the first sixteen-row step needs its eight probabilities");
  auto half_step = [&](f32x16& cur, f32x16& nxt, int it, auto j_c, auto hh_c) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value, hh = decltype(hh_c)::value;
    constexpr int BNX = B_USE + (hh ? (J + 1) % 4 : J) * TB;  // B tile of the next half
    constexpr int CF = C_FRAG + (J & 1) * TB;
    if constexpr (PRE) {
      // The same lazy rescale on relative scores: `cur` and mxn were computed against the present maximum.  The very
      // first half tile sets the maximum (whatever its sign; nothing is accumulated yet), later ones only raise it.
      const bool first = hh == 0 && it == 0;
      if (first || __builtin_amdgcn_ballot_w64(mxn > kLazy) != 0) {
        const float d = first ? mxn : fmaxf(mxn, 0.f);
        mrow += d;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          cur[r] -= d;
          negm[r] = -mrow;
        }
        if (!first) {
          const float alpha = __builtin_amdgcn_exp2f(-d);
          lsum *= alpha;
#pragma unroll
          for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
        }
      }
    } else if constexpr (INTER == kInterSoftmax) {
      // lazy rescale: raise the running maximum only when a row of the wave exceeds it by 2^kLazy
      if (__builtin_amdgcn_ballot_w64(mxn > mrow + kLazy) != 0) {
        const float mnew = fmaxf(mrow, mxn);
        const float alpha = __builtin_amdgcn_exp2f(mrow - mnew);
        mrow = mnew;
        lsum *= alpha;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[t][r] *= alpha;
      }
    }
    V8 fr[NG];
    auto fetch = [&](int k) __attribute__((always_inline)) {
      fr[k] = k < NS ? b_frag(BNX, hh ^ 1, k) : frag_rd(CF, (2 * hh + (k - NS) / NT) * NT + (k - NS) % NT);
    };
#pragma unroll
    for (int k = 0; k < kAhead; ++k) fetch(k);
    V8 pf[2];
#pragma unroll
    for (int k = 0; k < NG; ++k) {
      if (k + kAhead < NG) fetch(k + kAhead);
      __builtin_amdgcn_sched_barrier(0);
      if (k == 0) {
        const f32x16 z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        nxt = Elem<T>::mfma32(fr[k], af[k], PRE ? negm : z);
      } else if (k < NS) {
        nxt = Elem<T>::mfma32(fr[k], af[k], nxt);
      } else {
        o[(k - NS) % NT] = Elem<T>::mfma32(fr[k], pf[(k - NS) / NT], o[(k - NS) % NT]);
      }
      if constexpr (INTER == kInterSoftmax) {
        if (k < NS) exp_range(cur, k * EA / NS, (k + 1) * EA / NS);
        else if (k < NS + NT) exp_range(cur, EA + (k - NS) * (16 - EA) / NT, EA + (k - NS + 1) * (16 - EA) / NT);
      }
      if (k == NS - 1) make_p(cur, 0, pf[0]);
      if (k == NS + NT - 1) make_p(cur, 1, pf[1]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (INTER == kInterSoftmax) {
      const int nt = hh ? it + 1 : it;  // tile of the next half
      if (ragged && nt == ntiles - 1) mask_tail(nxt, nt * kBN + 32 * (hh ^ 1));
      row_max(nxt);
    }
  };
  auto tile_step_pipe = [&](int it, auto j_c) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;
    constexpr int PAR = J & 1;
    V8 xb[NTR], xc[NTR];
    load_c(it + C_AHEAD, NCR == 4 ? (J + 3) % 4 : PAR);
    load_b(it + B_AHEAD, B_KL ? (PAR ^ 1) : (J + 3) % 4);
    if (B_KL) tr_read_b(B_LOAD + PAR * TB, xb);
    tr_read_c(C_RAW + (NCR == 4 ? (J + 1) % 4 : (PAR ^ 1)) * TB, xc);
    half_step(sa, sb, it, j_c, IntC<0>{});
    if (B_KL) tr_write(B_FRAG + ((J + 2) % 4) * TB, xb);
    tr_write(C_FRAG + (PAR ^ 1) * TB, xc);
    half_step(sb, sa, it, j_c, IntC<1>{});
    if (B_KL) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    else if (NCR == 4) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NLD) : "memory");
    else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLD) : "memory");
    __syncthreads();
  };

  // ---- prologue: first tiles in flight, first transposition(s), the late waves' first scores
  load_b(0, 0);
  load_b(1, 1);
  load_c(0, 0);
  load_c(1, 1);
  if (!B_KL) load_b(2, 2);
  if (NCR == 4) load_c(2, 2);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  {
    V8 x[NTR];
    tr_read_c(C_RAW, x);
    tr_write(C_FRAG, x);
    if (B_KL) {
      tr_read_b(B_LOAD, x);
      tr_write(B_FRAG, x);
      tr_read_b(B_LOAD + TB, x);
      tr_write(B_FRAG + TB, x);
      __syncthreads();
      load_b(2, 0);
    }
  }
  if (late) scores(IntC<B_USE>{});
  if constexpr (PIPE) {  // scores of the very first half
#pragma unroll
    for (int k = 0; k < NS; ++k) {
      const V8 bf = b_frag(B_USE, 0, k);
      if (k == 0) {
        const f32x16 z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        sa = Elem<T>::mfma32(bf, af[k], z);
      } else {
        sa = Elem<T>::mfma32(bf, af[k], sa);
      }
    }
    if constexpr (INTER == kInterSoftmax) {
      if (ragged && ntiles == 1) mask_tail(sa, 0);
      row_max(sa);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  if constexpr (PIPE) {
    for (int it = 0; it < ntiles; it += 4) {
      tile_step_pipe(it, IntC<0>{});
      if (it + 1 < ntiles) tile_step_pipe(it + 1, IntC<1>{});
      if (it + 2 < ntiles) tile_step_pipe(it + 2, IntC<2>{});
      if (it + 3 < ntiles) tile_step_pipe(it + 3, IntC<3>{});
    }
  } else {
    for (int it = 0; it < ntiles; it += 4) {
      tile_step(it, IntC<0>{});
      if (it + 1 < ntiles) tile_step(it + 1, IntC<1>{});
      if (it + 2 < ntiles) tile_step(it + 2, IntC<2>{});
      if (it + 3 < ntiles) tile_step(it + 3, IntC<3>{});
    }
  }

  // ---- epilogue: normalise (softmax), cast, store: by rows through LDS (free by now) where the output allows
  // (store_tile_rows), else 4 contiguous columns per lane from registers
  const bool by_rows = !p.out_f32 && (N & 7) == 0 && (p.f_rs & 7) == 0 && (p.f_bs & 7) == 0 && (p.f_bs2 & 7) == 0 &&
                       (reinterpret_cast<size_t>(p.f) & 15) == 0;  // wave-uniform
  static_assert(8 * (32) * tile_row_bytes<D>() <= bmm_chain8_lds_bytes<D, B_KL>(), "the parked rows need the staged tiles' LDS");
  if (by_rows) {
    // every wave is done with the staged tiles, and the direct loads still in flight (the tiles past the last one:
    // zeros) have landed -- they would otherwise fall on the rows parked below
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    wg_sync();
  }
  char* const tw = smem_raw + wave * 32 * tile_row_bytes<D>();
  float inv = 1.f;
  if constexpr (INTER == kInterSoftmax) inv = 1.f / pair_sum(lsum);
  // lane coordinates taken afresh: values kept from the prologue for this would sit in registers (or spill)
  // through the whole walk
  int lane_e = threadIdx.x & 63;
  asm volatile("" : "+v"(lane_e));
  const int ln_e = lane_e & 31, g_e = lane_e >> 5;
  const int row = m_wave + ln_e;
  if (by_rows || row < M) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int n = 32 * t + 8 * q4 + 4 * g_e;
        if (!by_rows && n >= N) continue;
        float v0 = o[t][4 * q4 + 0] * inv, v1 = o[t][4 * q4 + 1] * inv;
        float v2 = o[t][4 * q4 + 2] * inv, v3 = o[t][4 * q4 + 3] * inv;
        if (INTER != kInterSoftmax && p.relu_out) { v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); v2 = fmaxf(v2, 0.f); v3 = fmaxf(v3, 0.f); }
        const long long off = zo * p.f_bs2 + zi * p.f_bs + (long long)row * p.f_rs + n;
        if (p.out_f32) {
          f32x4 w = {v0, v1, v2, v3};
          *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.f) + off) = w;
        } else {
          V2 a0 = cvt2<T>(v0, v1), a1 = cvt2<T>(v2, v3);
          V4 w = {a0[0], a0[1], a1[0], a1[1]};
          if (by_rows) *reinterpret_cast<V4*>(tw + ln_e * tile_row_bytes<D>() + n * 2) = w;
          else *reinterpret_cast<V4*>(reinterpret_cast<T*>(p.f) + off) = w;
        }
      }
  }
  if (by_rows)
    store_tile_rows<T, D, 32>(tw, reinterpret_cast<T*>(p.f) + zo * p.f_bs2 + zi * p.f_bs + (long long)m_wave * p.f_rs, p.f_rs,
                              M - m_wave, N, lane_e);
#else
  (void)p;
#endif
}

template <typename T, int D, int INTER, bool B_KL, bool PIPE = false>
hipError_t launch_bmm_chain8(const BmmChainArgs& args, hipStream_t stream) {
  constexpr int lds = bmm_chain8_lds_bytes<D, B_KL>();
  auto kern = bmm_chain8_kernel<T, D, INTER, B_KL, PIPE>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  const unsigned grid = (unsigned)args.mblocks * (unsigned)args.batch;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, stream, args);
  return hipGetLastError();
}

}  // namespace ditto
