// Fused two-contraction chain  F = epilogue(inter(A.B).C)  for fp16 / bf16 on gfx950.
//
// One kernel covers the reference's GEMM->GEMM chain (inter = cast / relu;
// benchmark/chimera/cuda/bmm_bmm_cuda.py:69-149) and its BMM->softmax->BMM chain
// (python/ditto/auto_compute/nn/functional/bmm_chain.py:5-105).  Where the
// reference's generated kernel stores the first accumulator tile to shared memory as
// fp32, re-reads it, exponentiates, re-writes it as fp16 and re-loads it into
// fragments, then leaves the divide to a second launch over an fp32 HBM buffer
// (evaluation/asplos/ncu_summary_chimera_bmm_softmax_bmm.txt:26-72,556-561), here
// the first contraction is computed TRANSPOSED (D^T = B^T.A^T) so that its MFMA
// accumulator registers already have the layout of the second contraction's
// B operand (F^T = C^T.P^T): the intermediate never leaves VGPRs.
//
// Work split: a workgroup of 4 waves (one per SIMD) owns 128*QT rows of A for one batch
// entry; each wave owns 32*QT rows and keeps their A fragments in VGPRs for the whole
// kernel.  The L axis is walked in steps of 64.  B and C tiles go from global memory
// straight into LDS (buffer_load ... lds, 16 bytes per lane, no staging registers; rows and
// columns outside the matrices read as zero through the buffer range check), double
// buffered, one barrier per step, shared by the 4 waves.  Tiles are stored unpadded with the
// 16-byte chunk index of each row XOR-swizzled so that both the plain 16-byte row reads and
// the transposing reads (ds_read_b64_tr_b16) are bank-conflict free.
//
// Software pipeline (one wave per SIMD, so overlap must come from within the wave): while
// the MFMA pipe computes the scores of step i+1, the VALU exponentiates the scores of step
// i; while it accumulates P(i).C(i), the VALU packs P(i) and takes the row maximum of step
// i+1.  The two score buffers alternate by unrolling the step loop twice.
#pragma once
#include "common.h"

namespace ditto {

struct BmmChainArgs {
  const void* a;
  const void* b;
  const void* c;
  void* f;
  long long a_bs, b_bs, c_bs, f_bs;  // batch strides, elements (inner level)
  long long a_bs2, b_bs2, c_bs2, f_bs2;  // outer-level batch strides
  int batch_inner;                   // entries of the inner batch level (= batch: single level)
  int a_rs, b_rs, c_rs, f_rs;        // row strides, elements
  int M, N, K, L, batch;
  int mblocks;       // workgroups per batch entry
  int mblocks3;      // 16x16x32-MFMA kernel: how many of them, the first ones, have 384 rows (the others 256)
  float scale_log2;  // softmax: scale * log2(e)
  int relu;          // inter = relu instead of cast (non-softmax kernels)
  int relu_out;      // ReLU on the second accumulator before the final cast (non-softmax kernels)
  int out_f32;       // write F as fp32 instead of T
};

template <int V>
struct IntC {
  static constexpr int value = V;
};

constexpr int kInterCast = 0;
constexpr int kInterSoftmax = 2;

constexpr int kBN = 64;        // L step
constexpr int kNW = 4;         // waves per workgroup
constexpr float kLazy = 8.0f;  // log2 of the slack allowed before the running maximum is raised

template <int D>
__host__ __device__ constexpr int bmm_chain_lds_bytes() {
  return (4 + 2) * kBN * D * 2;  // four B tiles, two C tiles, 16-bit elements
}

// XOR applied to the 16-byte chunk index of a row of an unpadded LDS tile.
//   row-read tiles (one 16-byte read per lane, consecutive lanes = consecutive rows):
//     16 consecutive rows must hit 16 different chunk slots of a 256-byte bank window
//   transpose-read tiles (ds_read_b64_tr_b16: 16 lanes read 4 rows x 32 bytes):
//     4 consecutive rows x 4 chunks must hit different slots
template <int CPR>  // chunks per row: 16 (256-byte rows) or 8 (128-byte rows)
__device__ __forceinline__ int swz_rowread(int row) {
  return CPR == 16 ? (row & 15) : ((row ^ (row >> 3)) & 7);
}
template <int CPR>
__device__ __forceinline__ int swz_trread(int row) {
  return CPR == 16 ? 4 * (row & 3) : 4 * ((row >> 1) & 1);
}

template <typename T, int D, int QT, int INTER, bool B_KL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void bmm_chain_kernel(BmmChainArgs p) {
  // The body uses device-only types (buffer resources); the host pass only needs the stub.
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  typedef typename Elem<T>::v2 V2;
  constexpr int BM = kNW * 32 * QT;
  constexpr int TILE = kBN * D;                 // elements per staged tile (B and C alike)
  constexpr int B_RB = B_KL ? kBN * 2 : D * 2;  // bytes per LDS row of the B tile
  constexpr int B_CPR = B_RB / 16;
  constexpr int C_RB = D * 2;
  constexpr int C_CPR = C_RB / 16;
  constexpr int NLD = TILE * 2 / 1024 / kNW;    // direct-load instructions per wave per tile
  static_assert(NLD >= 1, "tile too small");

  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  // B tiles [4][TILE] at byte 0, C tiles [2][TILE] at byte 4*TILE*2.  Tile t of B lives in
  // buffer t%4 and tile t of C in buffer t%2; the tile loop is unrolled four times so that every
  // buffer address is a compile-time constant and folds into the LDS instructions' offsets.
  constexpr int C_BASE = 4 * TILE * 2;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int i16 = lane & 15, h = (lane >> 4) & 1;

  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
  const int mb = lid % p.mblocks;
  const int bz = lid / p.mblocks;
  // batch entry bz = zo * batch_inner + zi
  const int zo = bz / p.batch_inner, zi = bz - zo * p.batch_inner;
  const T* __restrict__ Ag = reinterpret_cast<const T*>(p.a) + zo * p.a_bs2 + zi * p.a_bs;
  const T* Bg = reinterpret_cast<const T*>(p.b) + zo * p.b_bs2 + zi * p.b_bs;
  const T* Cg = reinterpret_cast<const T*>(p.c) + zo * p.c_bs2 + zi * p.c_bs;
  const int m_wave = mb * BM + wave * 32 * QT;
  const int M = p.M, N = p.N, K = p.K, L = p.L;

  // ---- buffer resources over this batch entry's B and C (reads past the end return 0)
  const unsigned b_bytes = (unsigned)(B_KL ? ((long long)(K - 1) * p.b_rs + L) : ((long long)(L - 1) * p.b_rs + K)) * 2u;
  const unsigned c_bytes = (unsigned)((long long)(L - 1) * p.c_rs + N) * 2u;
  const i32x4 b_rsrc = make_rsrc(Bg, b_bytes);
  const i32x4 c_rsrc = make_rsrc(Cg, c_bytes);
  const unsigned lds0 = (unsigned)(size_t)(DITTO_LDS char*)smem_raw;  // LDS byte address of the tiles

  // ---- per-lane source offsets of the direct loads.  Load q of this wave fills the LDS
  // bytes [1024*(NLD*wave + q), +1024): lane -> (row, physical chunk) -> swizzled source.
  int b_voff[NLD], c_voff[NLD];
  int b_col[NLD];  // B_KL only: first l column (within the tile) the lane loads
#pragma unroll
  for (int q = 0; q < NLD; ++q) {
    const int gi = NLD * wave + q;
    {
      const int row = gi * (64 / B_CPR) + lane / B_CPR, pc = lane % B_CPR;
      if (B_KL) {
        const int cl = pc ^ swz_trread<B_CPR>(row);  // rows are k, columns l
        b_col[q] = cl * 8;
        b_voff[q] = row < K ? (row * p.b_rs + cl * 8) * 2 : (int)b_bytes;
      } else {
        const int cl = pc ^ swz_rowread<B_CPR>(row);  // rows are l, columns k
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
  // direct load q (of NLD) of this wave for B tile `tile` into buffer `buf`
  auto load_b1 = [&](int tile, int buf, int q) __attribute__((always_inline)) {
    const int l0 = tile * kBN;
    const int soff = B_KL ? l0 * 2 : l0 * p.b_rs * 2;
    // the whole offset goes into the per-lane operand: it is what the range check sees
    int vo = b_voff[q] + soff;
    if (B_KL) vo = (l0 + b_col[q] < L) ? vo : (int)b_bytes;  // columns past L are inside the buffer
    lds_dma_16(b_rsrc, (unsigned)vo, lds0 + (buf * TILE) * 2 + 1024 * (NLD * wave + q));
  };
  auto load_c1 = [&](int tile, int buf, int q) __attribute__((always_inline)) {
    const int soff = tile * kBN * p.c_rs * 2;
    lds_dma_16(c_rsrc, (unsigned)(c_voff[q] + soff), lds0 + C_BASE + (buf * TILE) * 2 + 1024 * (NLD * wave + q));
  };
  auto load_b = [&](int tile, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < NLD; ++q) load_b1(tile, buf, q);
  };
  auto load_c = [&](int tile, int buf) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < NLD; ++q) load_c1(tile, buf, q);
  };

  // ---- per-lane LDS read offsets (bytes, within one tile)
  // B operand of step st, L-tile i (A operand of D^T = B^T.A^T: rows l, 8 consecutive k)
  //   row-read layout: row 32i+ln, logical chunk 2st+g      -> (2st) ^ (g ^ swz(ln))
  //   tr-read  layout: rows k = 16st+8g+(i16>>2)+{0,4}, chunk 4i+2h+((i16&3)>>1), +8*(i16&1)
  const int b_rd = B_KL ? ((8 * g + (i16 >> 2)) * B_RB + (2 * h + ((i16 & 3) >> 1)) * 16 + 8 * (i16 & 1))
                        : (ln * B_RB);
  // C operand of step u, N-tile t (A operand of F^T = C^T.P^T: rows n, k = l permuted):
  //   rows l = 16u + 4g + (i16>>2) + {0,8}, chunk 4t + 2h + ((i16&3)>>1), +8*(i16&1)
  const int c_rd = (4 * g + (i16 >> 2)) * C_RB + (2 * h + ((i16 & 3) >> 1)) * 16 + 8 * (i16 & 1);
  // Per-lane byte addresses, loop invariant; everything else is a compile-time offset.
  constexpr int NS = D / 16;
  int b_ad[2][NS], c_ad[D / 32];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int x = B_KL ? swz_trread<B_CPR>(i16 >> 2) : (g ^ swz_rowread<B_CPR>(32 * i + ln));
#pragma unroll
    for (int st = 0; st < NS; ++st) b_ad[i][st] = b_rd + (B_KL ? ((4 * i) ^ x) : ((2 * st) ^ x)) * 16;
  }
#pragma unroll
  for (int t = 0; t < D / 32; ++t) c_ad[t] = c_rd + ((4 * t) ^ swz_trread<C_CPR>(i16 >> 2)) * 16;

  // ---- A fragments (B operand of D^T = B^T.A^T): lane holds A[row][16s + 8g .. +7]
  V8 af[QT][D / 16];
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    const int row = m_wave + 32 * j + ln;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
      const int col = 16 * s + 8 * g;
      V8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (row < M && col < K) v = *reinterpret_cast<const V8*>(Ag + (long long)row * p.a_rs + col);
      af[j][s] = v;
    }
  }

  // ---- accumulators of F^T: o[t][j][r] = F^T[32t + 8(r/4) + 4g + r%4][32j + ln]
  f32x16 o[D / 32][QT];
#pragma unroll
  for (int t = 0; t < D / 32; ++t)
#pragma unroll
    for (int j = 0; j < QT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[t][j][r] = 0.f;
  // Softmax state per A-row tile j (one row per lane pair): running maximum mrow (exp2 domain),
  // partial row sum lsum, and mxn = scaled row maximum of the half tile about to be consumed.
  // Scores are raw dot products; p = exp2(s*c2 - mrow).
  float mrow[QT], lsum[QT], mxn[QT];
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    mrow[j] = -INFINITY;
    lsum[j] = 0.f;
    mxn[j] = -INFINITY;
  }
  const float c2 = p.scale_log2;
  const int ntiles = (L + kBN - 1) / kBN;
  const bool ragged = (L % kBN) != 0;

  // Scores are produced and consumed in HALF steps of 32 rows of the L tile: s[j] is the
  // transposed score tile (32 l x 32 m) of A-row tile j.
  // scores of rows past L are masked out (softmax only; other chains see zero operands)
  auto mask_tail = [&](f32x16 (&s)[QT], int l0) __attribute__((always_inline)) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int l = l0 + 8 * (r >> 2) + 4 * g + (r & 3);
      const int gone = (L - 1 - l) >> 31;  // all ones where l >= L
#pragma unroll
      for (int j = 0; j < QT; ++j) s[j][r] = neg_inf_where(s[j][r], gone);
    }
  };
  // scaled row maximum of a finished half tile (pair of half-waves combined)
  auto row_max = [&](f32x16 (&s)[QT]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      float mx = s[j][0];
#pragma unroll
      for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s[j][r]);
      mxn[j] = pair_max(mx) * c2;
    }
  };
  // Lazy rescale: the running maximum only has to bound the scores well enough that exp2
  // cannot overflow, so it is raised (and the accumulators rescaled) only when some row of
  // the wave exceeds it by more than 2^kLazy.  Rows keep a stale maximum otherwise; the
  // final division by the row sum cancels it exactly.
  auto maybe_rescale = [&](f32x16 (&cur)[QT]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      if (__builtin_amdgcn_ballot_w64(mxn[j] > mrow[j] + kLazy) != 0) {
        const float mnew = fmaxf(mrow[j], mxn[j]);
        const float alpha = __builtin_amdgcn_exp2f(mrow[j] - mnew);
        mrow[j] = mnew;
        lsum[j] *= alpha;
#pragma unroll
        for (int t = 0; t < D / 32; ++t)
#pragma unroll
          for (int r = 0; r < 16; ++r) o[t][j][r] *= alpha;
      }
    }
  };
  // exponentials of registers [r0, r0 + n) of the half tile
  auto exp_slice = [&](f32x16 (&s)[QT], int r0, int n) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < QT; ++j)
#pragma unroll
      for (int e = 0; e < n; ++e)
        s[j][r0 + e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j][r0 + e], c2, -mrow[j]));
  };
  // ---- operand fragments read from LDS
  // B fragment of MFMA group st for rows 32i..32i+31 of the L tile at byte offset `off`
  auto b_frag = [&](int off, int i, int st) __attribute__((always_inline)) -> V8 {
    if (B_KL) {
      const char* q = smem_raw + b_ad[i][st] + (off + 16 * st * B_RB);
      V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(q));
      V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(q + 4 * B_RB));
      return concat4<V4, V8>(lo, hi);
    }
    return *reinterpret_cast<const V8*>(smem_raw + b_ad[i][st] + (off + 32 * i * B_RB));
  };
  // C fragment of N tile t for rows 16u..16u+15 of the L tile at byte offset `off`
  auto c_frag = [&](int off, int u, int t) __attribute__((always_inline)) -> V8 {
    const char* q = smem_raw + c_ad[t] + (off + 16 * u * C_RB);
    V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(q));
    V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(q + 8 * C_RB));
    return concat4<V4, V8>(lo, hi);
  };
  // P fragment (B operand of the second contraction) of 16 rows of the L tile: registers
  // 8(u%2) .. 8(u%2)+7 of the half tile, cast; the row sum is taken over the ROUNDED
  // probabilities, i.e. exactly the values that enter the second contraction
  auto p_frag = [&](f32x16 (&s)[QT], int u, V8 (&pf)[QT]) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < QT; ++j) {
      const int r0 = 8 * (u & 1);
      float v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        v[e] = s[j][r0 + e];
        if (INTER != kInterSoftmax && p.relu) v[e] = fmaxf(v[e], 0.f);
      }
      V2 p0 = cvt2<T>(v[0], v[1]), p1 = cvt2<T>(v[2], v[3]), p2 = cvt2<T>(v[4], v[5]), p3 = cvt2<T>(v[6], v[7]);
      if constexpr (INTER == kInterSoftmax) {
        lsum[j] = Elem<T>::add_pair(p0, lsum[j]);
        lsum[j] = Elem<T>::add_pair(p1, lsum[j]);
        lsum[j] = Elem<T>::add_pair(p2, lsum[j]);
        lsum[j] = Elem<T>::add_pair(p3, lsum[j]);
      }
      V8 w = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
      pf[j] = w;
    }
  };

  // One pipelined half step: consumes the finished scores `cur` (half hh of L tile `it`) and
  // produces `nxt`, the scores of the following half (half 1 of the same tile, or half 0 of
  // tile it+1).  Past the last tile the MFMAs run on a resident but stale B buffer and their
  // result is dropped, which keeps the half step straight-line code.
  //
  // The half step is a sequence of NG MFMA groups, each fed by one LDS fragment: D/16 groups
  // of the first contraction (scores of the next half) followed by D/16 groups of the second
  // (2 sixteen-row steps x D/32 column tiles).  Fragments are fetched kAhead groups before
  // they are used so that the LDS latency is covered by the MFMAs of the groups in between;
  // the exponentials of `cur` are spread over the first-contraction groups.
  constexpr int NG = 2 * NS, kAhead = 2;
  auto half_step = [&](f32x16 (&cur)[QT], f32x16 (&nxt)[QT], int it, auto bi_c, auto hh_c) __attribute__((always_inline)) {
    constexpr int BI = decltype(bi_c)::value, hh = decltype(hh_c)::value;  // B buffer of tile it; half
    const int nt = hh ? it + 1 : it;  // tile of the next half
    constexpr int bs_next = ((hh ? (BI + 1) & 3 : BI) * TILE) * 2;
    constexpr int cs_cur = C_BASE + ((BI & 1) * TILE) * 2;
    if constexpr (INTER == kInterSoftmax) maybe_rescale(cur);
    V8 fr[NG];
    auto fetch = [&](int k) __attribute__((always_inline)) {
      // second contraction groups run N tile by N tile, two sixteen-row steps each
      fr[k] = k < NS ? b_frag(bs_next, hh ^ 1, k) : c_frag(cs_cur, 2 * hh + (k - NS) % 2, (k - NS) / 2);
    };
#pragma unroll
    for (int k = 0; k < kAhead; ++k) fetch(k);
    V8 pf[2][QT];
#pragma unroll
    for (int k = 0; k < NG; ++k) {
      if (k + kAhead < NG) fetch(k + kAhead);
      if (hh == 0) {
        // the direct loads for two tiles ahead are spread over the groups of the first half
        // step (a burst of them would hold up the wave's single instruction stream)
        constexpr int NL2 = 2 * NLD, EVERY = NG / NL2 > 0 ? NG / NL2 : 1;
        if (k % EVERY == 0 && k / EVERY < NL2) {
          const int q = k / EVERY;
          if (q < NLD) load_b1(it + 2, (BI + 2) & 3, q);
          else load_c1(it + 1, (BI + 1) & 1, q - NLD);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      if (k < NS) {
#pragma unroll
        for (int j = 0; j < QT; ++j) {
          if (k == 0) {
            const f32x16 z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
            nxt[j] = Elem<T>::mfma32(fr[k], af[j][k], z);
          } else {
            nxt[j] = Elem<T>::mfma32(fr[k], af[j][k], nxt[j]);
          }
        }
        if constexpr (INTER == kInterSoftmax) exp_slice(cur, (16 / NS) * k, 16 / NS);
      } else {
        const int uu = (k - NS) % 2, t = (k - NS) / 2;
        if (k == NS) {
          p_frag(cur, 2 * hh, pf[0]);
          p_frag(cur, 2 * hh + 1, pf[1]);
        }
#pragma unroll
        for (int j = 0; j < QT; ++j) o[t][j] = Elem<T>::mfma32(fr[k], pf[uu][j], o[t][j]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (INTER == kInterSoftmax) {
      if (ragged && nt == ntiles - 1) mask_tail(nxt, nt * kBN + 32 * (hh ^ 1));
      row_max(nxt);
    }
  };
  // scores of the very first half (prologue)
  auto first_half = [&](f32x16 (&s)[QT]) __attribute__((always_inline)) {
#pragma unroll
    for (int st = 0; st < NS; ++st) {
      const V8 bf = b_frag(0, 0, st);
#pragma unroll
      for (int j = 0; j < QT; ++j) {
        if (st == 0) {
          const f32x16 z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
          s[j] = Elem<T>::mfma32(bf, af[j][st], z);
        } else {
          s[j] = Elem<T>::mfma32(bf, af[j][st], s[j]);
        }
      }
    }
  };

  // ---- prologue: B(0), C(0), B(1) in flight; scores of the first half
  load_b(0, 0);
  load_c(0, 0);
  load_b(1, 1);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  f32x16 sa[QT], sb[QT];
  first_half(sa);
  if constexpr (INTER == kInterSoftmax) {
    if (ragged && ntiles == 1) mask_tail(sa, 0);
    row_max(sa);
  }

  // One L tile: loads two tiles ahead (B(it+2) replaces B(it-2), C(it+1) replaces C(it-1); both
  // were released by earlier barriers; tiles past the end are entirely out of range and load
  // zeros), then the two pipelined half steps, then the barrier that publishes the loads.
  auto tile_step = [&](int it, auto bi_c) __attribute__((always_inline)) {
    constexpr int BI = decltype(bi_c)::value;
    half_step(sa, sb, it, bi_c, IntC<0>{});
    half_step(sb, sa, it, bi_c, IntC<1>{});
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  for (int it = 0; it < ntiles; it += 4) {
    tile_step(it, IntC<0>{});
    if (it + 1 < ntiles) tile_step(it + 1, IntC<1>{});
    if (it + 2 < ntiles) tile_step(it + 2, IntC<2>{});
    if (it + 3 < ntiles) tile_step(it + 3, IntC<3>{});
  }

  // ---- epilogue: normalise (softmax), cast, store: by rows through LDS (free by now) where the output allows
  // (store_tile_rows), else 4 contiguous columns per lane from registers
  const bool by_rows = !p.out_f32 && (N & 7) == 0 && (p.f_rs & 7) == 0 && (p.f_bs & 7) == 0 && (p.f_bs2 & 7) == 0 &&
                       (reinterpret_cast<size_t>(p.f) & 15) == 0;  // wave-uniform
  static_assert(4 * (32 * QT) * tile_row_bytes<D>() <= bmm_chain_lds_bytes<D>(), "the parked rows need the staged tiles' LDS");
  if (by_rows) {
    // every wave is done with the staged tiles, and the direct loads still in flight (the tiles past the last one:
    // zeros) have landed -- they would otherwise fall on the rows parked below
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    wg_sync();
  }
  char* const tw = smem_raw + wave * (32 * QT) * tile_row_bytes<D>();
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    float inv = 1.f;
    if constexpr (INTER == kInterSoftmax) inv = 1.f / pair_sum(lsum[j]);
    const int row = m_wave + 32 * j + ln;
    if (!by_rows && row >= M) continue;
#pragma unroll
    for (int t = 0; t < D / 32; ++t)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int n = 32 * t + 8 * q4 + 4 * g;
        if (!by_rows && n >= N) continue;
        float v0 = o[t][j][4 * q4 + 0] * inv, v1 = o[t][j][4 * q4 + 1] * inv;
        float v2 = o[t][j][4 * q4 + 2] * inv, v3 = o[t][j][4 * q4 + 3] * inv;
        if (INTER != kInterSoftmax && p.relu_out) { v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); v2 = fmaxf(v2, 0.f); v3 = fmaxf(v3, 0.f); }
        const long long off = zo * p.f_bs2 + zi * p.f_bs + (long long)row * p.f_rs + n;
        if (p.out_f32) {
          f32x4 w = {v0, v1, v2, v3};
          *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.f) + off) = w;
        } else {
          V2 a0 = cvt2<T>(v0, v1), a1 = cvt2<T>(v2, v3);
          V4 w = {a0[0], a0[1], a1[0], a1[1]};
          if (by_rows) *reinterpret_cast<V4*>(tw + (32 * j + ln) * tile_row_bytes<D>() + n * 2) = w;
          else *reinterpret_cast<V4*>(reinterpret_cast<T*>(p.f) + off) = w;
        }
      }
  }
  if (by_rows)
    store_tile_rows<T, D, 32 * QT>(tw, reinterpret_cast<T*>(p.f) + zo * p.f_bs2 + zi * p.f_bs + (long long)m_wave * p.f_rs,
                                   p.f_rs, M - m_wave, N, lane);
#else
  (void)p;
#endif
}

// Host-side launcher for one instantiation.
template <typename T, int D, int QT, int INTER, bool B_KL>
hipError_t launch_bmm_chain(const BmmChainArgs& args, hipStream_t stream) {
  constexpr int lds = bmm_chain_lds_bytes<D>();
  auto kern = bmm_chain_kernel<T, D, QT, INTER, B_KL>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  const unsigned grid = (unsigned)args.mblocks * (unsigned)args.batch;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, args);
  return hipGetLastError();
}

}  // namespace ditto
