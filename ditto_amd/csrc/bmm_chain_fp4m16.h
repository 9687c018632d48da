// Four-wave fused two-contraction chain on the 16x16x32 MFMA with 64-row workgroups, head dimension up to 64
// (see bmm_chain_fp.h for the chain and the transposed formulation, bmm_chain_fp8m16.h for the operand layouts
// of v_mfma_f32_16x16x32 and the register-resident hand-over between the two contractions).
//
// Why another workgroup shape: short sequences.  96 heads of 512 rows are 192 workgroups of 256 rows, or 384 of
// 128: neither fills 256 compute units evenly (a quarter of them idle, or half of them with twice the work of the
// others).  In 64-row workgroups the same problem is 768 = 3 x 256 workgroups of four waves, three per compute unit
// (48 KB of LDS each, at most 168 registers per lane), three waves on every SIMD.
//
// Two forms (KSPLIT):
//   1: a wave owns ONE 16-row tile and all 64 keys of a tile.  Least to do before the first and after the last step,
//      the faster form up to about 1000 keys.  Its price is LDS traffic: every operand fragment feeds one MFMA, three
//      workgroups read 192 KB and the direct loads write 48 KB per step and compute unit, three quarters of the
//      step's cycles at 256 / 128 bytes per cycle (and, on N(0,1) operands, a clock of 1.7 GHz: the device runs this
//      kernel against its power limit, like the long-sequence kernels).
//   2: the workgroup is split two ways in rows and two ways in KEYS: wave w owns rows 32 (w % 2) .. + 31 (two 16-row
//      tiles: every fragment read feeds two MFMAs, half the LDS reads) and, of every 64-key tile, keys
//      32 (w / 2) .. + 31: the same sixteen MFMAs per wave and step.  Each wave runs its own online softmax over its
//      keys; the two halves of a row are merged once, at the end, through LDS (each wave of a pair finishes one of the
//      pair's two row tiles).  A step is a tenth shorter, the merge costs about what six steps save.
//
// LDS: a ring of three B tiles ([64 l][D k] as loaded, or [D k][64 l] when B is stored [K][L]) and three C tiles
// ([64 l][D n] as loaded).  A wave reads its C^T fragments from the raw tile with two transposing reads
// (ds_read_b64_tr_b16) per fragment, and its B fragments likewise when B is stored [K][L]: the contraction index of
// a fragment then runs 4 q .. + 3, 16 + 4 q .. + 3 within a step of 32, and the A fragments are loaded in that order.
//
// Softmax: the optimistic walk of bmm_chain_fp8m16.h (the reference exponent of a row is the maximum of the wave's
// first keys; the lane's partial row SUM is watched once per tile and the reference raised by whole binary orders
// when it passes a limit; a sum that ends up infinite or NaN sends the workgroup through the exact walk), for bf16
// and for fp16: an fp16 probability overflows at 2^16, so the limit is 2^8 there and a row whose scores climb by
// more than 2^8 within one tile takes the second walk.  fp16 also uses the pre-scaled form of the pipelined
// eight-wave kernel: A is multiplied by scale * log2(e) once and every score tile starts from minus the reference
// exponent, so a score costs its v_exp_f32 and nothing else.
#pragma once
#include "bmm_chain_fp8m16.h"

namespace ditto {

constexpr int kRing4m16 = 3;

// XOR applied to the 16-byte chunk index of a 128-byte tile row in this kernel.  LDS serves 256 bytes per cycle from
// 64 banks; measured with eight waves reading at once, a 16-byte read per lane with lanes (c, q) -> (row c, chunk q)
// takes 4 cycles under the first swizzle and 8 under the row-read swizzle of the 32-row kernels; the transposing read
// (lanes (c, q) -> row 4 q + c / 4, 8 bytes at column 4 (c % 4)) takes 2.3 cycles under the second and 4 under theirs.
__device__ __forceinline__ int swz4m16_rows(int row) { return (row >> 1) & 7; }
__device__ __forceinline__ int swz4m16_tr(int row) { return 2 * ((row >> 1) & 3); }

template <int D>
__host__ __device__ constexpr int bmm_chain4m16_lds_bytes() {
  return 2 * kRing4m16 * kBN * D * 2 + 64;  // the tiles and the flag of the optimistic walk
}

template <typename T, int D, int INTER, int KSPLIT, bool B_KL>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void bmm_chain4m16_kernel(BmmChainArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  typedef typename Elem<T>::v2 V2;
  static_assert(D == 64, "128-byte tile rows");
  constexpr int NW = 4;
  static_assert(KSPLIT == 1 || KSPLIT == 2, "one or two key halves");
  constexpr int RT = KSPLIT;             // 16-row tiles per wave
  constexpr int NI = kBN / 16 / KSPLIT;  // 16-key tiles per wave and step
  constexpr int NH = NI / 2;             // 32-key halves per wave and step (one second-contraction operand each)
  constexpr int NR = kRing4m16;
  constexpr int TB = kBN * D * 2;        // bytes per tile
  constexpr int RB = D * 2;              // bytes per LDS row
  constexpr int CPR = RB / 16;           // 16-byte chunks per row
  constexpr int NS = D / 32;             // k steps of the first contraction
  constexpr int NTN = D / 16;            // column tiles of the second contraction
  constexpr int NLD = TB / 1024 / NW;    // direct loads per wave per tile
  constexpr int B_OFF = 0, C_OFF = NR * TB;
  constexpr bool kSoftmax = INTER == kInterSoftmax;
  constexpr bool PRE = kSoftmax && !Elem<T>::is_bf16;
  // a lane's partial row sum above which the reference exponent is raised
  constexpr float kLimit = Elem<T>::is_bf16 ? kSumLimitBf16 : kSumLimitF16;

  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // KSPLIT == 2: row half of the workgroup, key half of every tile; KSPLIT == 1: a wave owns one 16-row tile and all keys
  const int rh = KSPLIT == 2 ? (wave & 1) : wave, kh = KSPLIT == 2 ? (wave >> 1) : 0;
  const int c16 = lane & 15, q = lane >> 4;

  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
  const int mb = lid % p.mblocks;
  const int bz = lid / p.mblocks;
  const int zo = bz / p.batch_inner, zi = bz - zo * p.batch_inner;
  const T* __restrict__ Ag = reinterpret_cast<const T*>(p.a) + zo * p.a_bs2 + zi * p.a_bs;
  const T* Bg = reinterpret_cast<const T*>(p.b) + zo * p.b_bs2 + zi * p.b_bs;
  const T* Cg = reinterpret_cast<const T*>(p.c) + zo * p.c_bs2 + zi * p.c_bs;
  const int m_wave = mb * 64 + rh * (16 * RT);  // (either way 16 RT rows per unit of rh)
  const int M = p.M, N = p.N, K = p.K, L = p.L;

  const unsigned b_bytes = (unsigned)(B_KL ? ((long long)(K - 1) * p.b_rs + L) : ((long long)(L - 1) * p.b_rs + K)) * 2u;
  const unsigned c_bytes = (unsigned)((long long)(L - 1) * p.c_rs + N) * 2u;
  const i32x4 b_rsrc = make_rsrc(Bg, b_bytes);
  const i32x4 c_rsrc = make_rsrc(Cg, c_bytes);
  const unsigned lds0 = (unsigned)(size_t)(DITTO_LDS char*)smem_raw;

  // ---- A fragments first (their loads are the oldest in the vector-memory queue): lane holds
  // A[16 j + c][32 st + 8 q .. + 7]; with B stored [K][L] its fragments come out of transposing reads with the
  // contraction index in the order 4 q .. + 3, 16 + 4 q .. + 3 (like the C fragments), and A follows:
  // A[16 j + c][32 st + 4 q .. + 3] and A[16 j + c][32 st + 16 + 4 q .. + 3]
  V8 af[RT][NS];
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    const int row = m_wave + 16 * j + c16;
#pragma unroll
    for (int st = 0; st < NS; ++st) {
      if (B_KL) {
        const int col = 32 * st + 4 * q;
        V4 lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
        if (row < M && col < K) lo = *reinterpret_cast<const V4*>(Ag + (long long)row * p.a_rs + col);
        if (row < M && col + 16 < K) hi = *reinterpret_cast<const V4*>(Ag + (long long)row * p.a_rs + col + 16);
        af[j][st] = concat4<V4, V8>(lo, hi);
      } else {
        const int col = 32 * st + 8 * q;
        V8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (row < M && col < K) v = *reinterpret_cast<const V8*>(Ag + (long long)row * p.a_rs + col);
        af[j][st] = v;
      }
    }
  }

  // ---- per-lane source offsets of the direct loads: load i of this wave fills LDS bytes [1024 (NLD wave + i), + 1024)
  // of a tile, lane -> (row, physical chunk) -> swizzled source chunk
  int b_voff[NLD], c_voff[NLD];
  int b_col[NLD];  // B stored [K][L] only: first key (within the tile) the lane loads
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int gi = NLD * wave + i;
    const int row = gi * (64 / CPR) + lane / CPR, pc = lane % CPR;
    if (B_KL) {
      const int bl = pc ^ swz4m16_tr(row);  // rows are k, columns l
      b_col[i] = bl * 8;
      b_voff[i] = row < K ? (row * p.b_rs + bl * 8) * 2 : (int)b_bytes;
    } else {
      const int bl = pc ^ swz4m16_rows(row);  // rows are l, columns k
      b_col[i] = 0;
      b_voff[i] = bl * 8 < K ? (row * p.b_rs + bl * 8) * 2 : (int)b_bytes;
    }
    const int cl = pc ^ swz4m16_tr(row);    // rows are l, columns n
    c_voff[i] = cl * 8 < N ? (row * p.c_rs + cl * 8) * 2 : (int)c_bytes;
  }
  // tiles past the last one are out of range and load zeros
  const unsigned lds_wave = lds0 + 1024 * NLD * wave;  // this wave's share of a tile slot
  auto load_tile = [&](int tile, int buf) __attribute__((always_inline)) {
    int bo = B_KL ? tile * kBN * 2 : tile * kBN * p.b_rs * 2, co = tile * kBN * p.c_rs * 2;
    asm volatile("" : "+s"(bo), "+s"(co));
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      int vo = b_voff[i] + bo;
      if (B_KL) vo = (tile * kBN + b_col[i] < L) ? vo : (int)b_bytes;  // keys past L lie inside the buffer (the next row)
      lds_dma_16_at(b_rsrc, (unsigned)vo, lds_wave, B_OFF + buf * TB + 1024 * i);
    }
#pragma unroll
    for (int i = 0; i < NLD; ++i) lds_dma_16_at(c_rsrc, (unsigned)(c_voff[i] + co), lds_wave, C_OFF + buf * TB + 1024 * i);
  };

  // ---- per-lane LDS read addresses (bytes within a tile), loop invariant; the wave's key half is folded in
  // B fragment (16-row tile i of the key half, k step st): row 32 kh + 16 i + c, logical chunk 4 st + q; the swizzle
  // of that row does not depend on kh or i
  // B stored [K][L]: the tile is [k][64 l] and a fragment (tile i, k step st) is read like a C^T fragment:
  // rows 32 st + 4 q + {0..3} (and + 16) x columns 16 (2 kh + i) .. + 15
  constexpr int NBA = B_KL ? NI : NS;
  int b_ad[NBA];
  if (B_KL) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int row = 4 * q + (c16 >> 2);
      const int chunk = 2 * (NI * kh + i) + ((c16 & 3) >> 1);
      b_ad[i] = row * RB + ((chunk ^ swz4m16_tr(row)) * 16) + 8 * (c16 & 1);
    }
  } else {
#pragma unroll
    for (int st = 0; st < NS; ++st) b_ad[st] = (32 * kh + c16) * RB + (((4 * st + q) ^ swz4m16_rows(c16)) * 16);
  }
  // C^T fragment (column tile t) of the key half: the 16 lanes of group q read rows 32 kh + 4 q + {0..3} (and + 16) x
  // columns 16 t .. + 15; lane s of the group points at row s / 4, 8 bytes at column 4 (s % 4).  The swizzle of a row
  // depends on row % 8 only.
  int c_ad[NTN];
#pragma unroll
  for (int t = 0; t < NTN; ++t) {
    const int row = 4 * q + (c16 >> 2);
    const int chunk = 2 * t + ((c16 & 3) >> 1);
    c_ad[t] = (32 * kh + row) * RB + ((chunk ^ swz4m16_tr(row)) * 16) + 8 * (c16 & 1) + C_OFF;
  }
  auto b_frag = [&](int buf, int i, int st) __attribute__((always_inline)) -> V8 {
    if (B_KL) {
      const char* a = smem_raw + b_ad[i % NBA] + (B_OFF + buf * TB + 32 * st * RB);
      V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(a));
      V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(a + 16 * RB));
      return concat4<V4, V8>(lo, hi);
    }
    return *reinterpret_cast<const V8*>(smem_raw + b_ad[st % NBA] + (B_OFF + buf * TB + 16 * i * RB));
  };
  auto c_frag = [&](int buf, int h, int t) __attribute__((always_inline)) -> V8 {
    const char* a = smem_raw + c_ad[t] + (buf * TB + 32 * h * RB);
    V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(a));
    V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(a + 16 * RB));
    return concat4<V4, V8>(lo, hi);
  };

  // The first tile's loads go out before anything waits for A: the wait the compiler puts in front of the first use of
  // the A fragments covers every load issued so far, so with A's loads, that wait and only then the tile's loads, a
  // workgroup started with two memory latencies in a row.  The fragments are used here (scaled, or merely named), so
  // that the wait falls between the first and the second tile's loads and does not take the second tile in as well.
  load_tile(0, 0);
#pragma unroll
  for (int j = 0; j < RT; ++j)
#pragma unroll
    for (int st = 0; st < NS; ++st) {
      if constexpr (PRE) {
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
          const V2 q2 = cvt2<T>((float)af[j][st][e] * p.scale_log2, (float)af[j][st][e + 1] * p.scale_log2);
          af[j][st][e] = q2[0];
          af[j][st][e + 1] = q2[1];
        }
      }
      asm volatile("" : "+v"(af[j][st]));
    }
  load_tile(1, 1);

  // ---- accumulators of F^T over the wave's keys: o[t][j][r] = F^T[16 t + 4 q + r][16 j + c]
  f32x4 o[NTN][RT];
  // softmax state of the lane's two rows (exp2 domain): reference exponent (the same in the four lanes of a row),
  // the lane's share of the row sum, and (pre-scaled form) four copies of minus the reference, the accumulator a
  // score tile starts from
  float mrow[RT], lsum[RT];
  // kSumMfma: the row sums come out of the matrix pipe instead: one more MFMA per operand, against a fragment of
  // ones, leaves the sum of the row's 32 probabilities in every register of ls[j] (all lanes of the row, no
  // exchange between lanes at the end), and the eight v_dot2c per lane and step go
#ifdef DITTO_4M16_SUM_VALU
  constexpr bool kSumMfma = false;
#else
  constexpr bool kSumMfma = kSoftmax;
#endif
  f32x4 ls[RT];
  V8 ones;
#pragma unroll
  for (int e = 0; e < 8; ++e) ones[e] = (T)1.0f;
  asm volatile("" : "+v"(ones));  // kept in vector registers: as a known constant it is rebuilt from scalar ones every tile
  auto row_part = [&](int j) __attribute__((always_inline)) -> float { return kSumMfma ? ls[j][0] : lsum[j]; };
  auto row_scale = [&](int j, float a) __attribute__((always_inline)) {
    if (kSumMfma) ls[j] *= a;
    else lsum[j] *= a;
  };
  // a lane's figure -> the row's (already the row's with kSumMfma)
  auto row_total = [&](float x) __attribute__((always_inline)) -> float { return kSumMfma ? x : quad_sum(x); };
  f32x4 negm[RT];
  const float c2 = p.scale_log2;
  const int ntiles = (L + kBN - 1) / kBN;
  const bool ragged = (L % kBN) != 0;
  int* const flag = reinterpret_cast<int*>(smem_raw + 2 * NR * TB);  // behind the tiles

  // One L tile.  J = it % 3 selects the ring slot (compile time).
  auto tile_step = [&](int it, auto j_c, auto safe_c) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;
    constexpr bool SAFE = decltype(safe_c)::value;
    // Tile it has landed (the loads of tile it + 1, issued a step ago, may stay in flight) and every wave is done
    // with tile it - 1, whose slot the loads below fill.
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NLD) : "memory");
    __syncthreads();
    load_tile(it + 2, (J + 2) % NR);

    // first contraction, transposed: s[i][j][r] = S^T[32 kh + 16 i + 4 q + r][16 j + c]
    // (k step outermost: consecutive MFMAs write different accumulators)
    f32x4 s[NI][RT];
#pragma unroll
    for (int st = 0; st < NS; ++st)
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const V8 bf = b_frag(J, i, st);
#pragma unroll
        for (int j = 0; j < RT; ++j) {
          if (st == 0) s[i][j] = Elem<T>::mfma16(bf, af[j][st], PRE ? negm[j] : f32x4{0.f, 0.f, 0.f, 0.f});
          else s[i][j] = Elem<T>::mfma16(bf, af[j][st], s[i][j]);
        }
      }
    if constexpr (kSoftmax) {
      if (ragged && it == ntiles - 1) {
        const int rem = L - it * kBN - 32 * kh - 4 * q;  // keys left, counted from the lane's first
#pragma unroll
        for (int i = 0; i < NI; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int gone = (rem - (16 * i + r) - 1) >> 31;  // all ones where 16 i + r >= rem
#pragma unroll
            for (int j = 0; j < RT; ++j) s[i][j][r] = neg_inf_where(s[i][j][r], gone);
          }
      }
      if (SAFE || it == 0) {
        float mx[RT];
#pragma unroll
        for (int j = 0; j < RT; ++j) {
          mx[j] = s[0][j][0];
#pragma unroll
          for (int i = 0; i < NI; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) mx[j] = fmaxf(mx[j], s[i][j][r]);
          if (!PRE) mx[j] *= c2;
        }
        if (it == 0) {
          // the first tile sets the reference; nothing is accumulated yet.  A wave none of whose keys exist (the upper
          // key half of a chain with at most 32 keys) takes zero: all its probabilities are exp2(-inf) = 0.
#pragma unroll
          for (int j = 0; j < RT; ++j) {
            float m0 = quad_max(mx[j]);
            if (!(m0 > -INFINITY)) m0 = 0.f;
            mrow[j] = m0;
            if (PRE) {
              negm[j] = f32x4{-m0, -m0, -m0, -m0};
#pragma unroll
              for (int i = 0; i < NI; ++i) s[i][j] -= m0;
            }
          }
        } else {
          bool vote = false;
#pragma unroll
          for (int j = 0; j < RT; ++j) vote = vote || (PRE ? mx[j] > kLazy : mx[j] > mrow[j] + kLazy);
          if (__builtin_amdgcn_ballot_w64(vote) != 0) {
            // exact walk: the reference follows the running maximum, lazily
#pragma unroll
            for (int j = 0; j < RT; ++j) {
              const float d = PRE ? fmaxf(quad_max(mx[j]), 0.f) : fmaxf(quad_max(mx[j]) - mrow[j], 0.f);
              const float alpha = __builtin_amdgcn_exp2f(-d);
              mrow[j] += d;
              row_scale(j, alpha);
#pragma unroll
              for (int t = 0; t < NTN; ++t) o[t][j] *= alpha;
              if (PRE) {
                negm[j] = f32x4{-mrow[j], -mrow[j], -mrow[j], -mrow[j]};
#pragma unroll
                for (int i = 0; i < NI; ++i) s[i][j] -= d;
              }
            }
          }
        }
      }
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < RT; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            s[i][j][r] = PRE ? __builtin_amdgcn_exp2f(s[i][j][r]) : __builtin_amdgcn_exp2f(__builtin_fmaf(s[i][j][r], c2, -mrow[j]));
    }
    // second contraction, 32 keys (half h) at a time: o[t][j] += C^T(half h, column tile t) . P^T(half h, row tile j);
    // operand slots 0..3 come from 16-key tile 2 h of the wave's keys, slots 4..7 from tile 2 h + 1; the row sum is
    // taken over the ROUNDED values, exactly what enters the MFMA
#pragma unroll
    for (int h = 0; h < NH; ++h) {
      V8 pf[RT];
#pragma unroll
      for (int j = 0; j < RT; ++j) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[e] = s[2 * h + (e >> 2)][j][e & 3];
          if (!kSoftmax && p.relu) v[e] = fmaxf(v[e], 0.f);
        }
        V2 p0 = cvt2<T>(v[0], v[1]), p1 = cvt2<T>(v[2], v[3]), p2 = cvt2<T>(v[4], v[5]), p3 = cvt2<T>(v[6], v[7]);
        if constexpr (kSoftmax && !kSumMfma) {
          lsum[j] = Elem<T>::add_pair(p0, lsum[j]);
          lsum[j] = Elem<T>::add_pair(p1, lsum[j]);
          lsum[j] = Elem<T>::add_pair(p2, lsum[j]);
          lsum[j] = Elem<T>::add_pair(p3, lsum[j]);
        }
        pf[j] = V8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
        if constexpr (kSumMfma) ls[j] = Elem<T>::mfma16(ones, pf[j], ls[j]);
      }
#pragma unroll
      for (int t = 0; t < NTN; ++t) {
        const V8 cf = c_frag(J, h, t);
#pragma unroll
        for (int j = 0; j < RT; ++j) o[t][j] = Elem<T>::mfma16(cf, pf[j], o[t][j]);
      }
    }
    if constexpr (kSoftmax && !SAFE) {
      // optimistic walk: once per tile, lower the scale of a row whose sum has passed the limit
      float smax = row_part(0);
#pragma unroll
      for (int j = 1; j < RT; ++j) smax = fmaxf(smax, row_part(j));
      if (__builtin_amdgcn_ballot_w64(smax > kLimit) != 0) {
#pragma unroll
        for (int j = 0; j < RT; ++j) {
          const float sref = kSumMfma ? ls[j][0] : quad_max(lsum[j]);  // the same in the four lanes of a row
          // (an infinite or NaN sum is left as it is: that is what the end of the walk looks for)
          const int e = (sref > kLimit && sref < INFINITY) ? ((__builtin_bit_cast(int, sref) >> 23) & 255) - 127 : 0;
          const float alpha = __builtin_bit_cast(float, (127 - e) << 23);  // 2^-e, exact
          mrow[j] += (float)e;
          if (PRE) negm[j] = f32x4{-mrow[j], -mrow[j], -mrow[j], -mrow[j]};
          row_scale(j, alpha);
#pragma unroll
          for (int t = 0; t < NTN; ++t) o[t][j] *= alpha;
        }
      }
    }
  };

  auto walk = [&](auto safe_c) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < RT; ++j) {
#pragma unroll
      for (int t = 0; t < NTN; ++t) o[t][j] = f32x4{0.f, 0.f, 0.f, 0.f};
      mrow[j] = 0.f;
      lsum[j] = 0.f;
      ls[j] = f32x4{0.f, 0.f, 0.f, 0.f};
      negm[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // (tiles 0 and 1 are in flight: issued by the caller)
    for (int it = 0; it < ntiles; it += 3) {
      tile_step(it, IntC<0>{}, safe_c);
      if (it + 1 < ntiles) tile_step(it + 1, IntC<1>{}, safe_c);
      if (it + 2 < ntiles) tile_step(it + 2, IntC<2>{}, safe_c);
    }
    // no direct load still on its way into LDS, every wave done with the tiles
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (kSoftmax && !decltype(safe_c)::value) {
      // a sum that is not finite in any lane of the workgroup sends all of it through the exact walk (the tiles are
      // the workgroup's common property); the flag lies behind the tiles and was cleared before the first barrier
      bool bad = false;
#pragma unroll
      for (int j = 0; j < RT; ++j) bad = bad || !(row_part(j) < INFINITY);
      if (__builtin_amdgcn_ballot_w64(bad) != 0 && lane == 0) *flag = 1;
    }
    wg_sync();
  };

  if (tid == 0) *flag = 0;
  walk(BoolC<false>{});
  if constexpr (kSoftmax) {
    if (__builtin_amdgcn_readfirstlane(*flag)) {
      load_tile(0, 0);
      load_tile(1, 1);
      walk(BoolC<true>{});
    }
  }

  // ---- KSPLIT == 2, the two key halves of a row meet: each wave of a pair finishes ONE of the pair's two row tiles
  // (tile kh) and hands the other tile's accumulators, sums and reference exponents to its partner (same lane, same
  // rows and columns) through LDS, [value][lane]
  constexpr int XCH = KSPLIT == 2 ? (NTN * 16 + 2 * 4) * 64 : 0;  // bytes per wave
  f32x4 oo[NTN];
  float inv = 1.f;
  if constexpr (KSPLIT == 2) {
    char* const xw = smem_raw + (wave ^ 2) * XCH + lane * 16;  // the partner's inbox
    char* const xr = smem_raw + wave * XCH + lane * 16;
#pragma unroll
    for (int t = 0; t < NTN; ++t) *reinterpret_cast<f32x4*>(xw + t * 1024) = kh ? o[t][0] : o[t][RT - 1];
    if constexpr (kSoftmax) {
      float* const xs = reinterpret_cast<float*>(smem_raw + (wave ^ 2) * XCH + NTN * 1024) + lane;
      xs[0] = kh ? row_part(0) : row_part(RT - 1);
      xs[64] = kh ? mrow[0] : mrow[RT - 1];
    }
    wg_sync();
    float fa = 1.f, fb = 1.f;
    if constexpr (kSoftmax) {
      const float* const xs = reinterpret_cast<const float*>(smem_raw + wave * XCH + NTN * 1024) + lane;
      // row sums of the two halves (a key half that holds a key has a sum of at least one: its reference is one of
      // its scores or lies below one; a half without keys has sum zero and takes no part)
      const float la = row_total(kh ? row_part(RT - 1) : row_part(0)), lb = row_total(xs[0]);
      const float ma = la > 0.f ? (kh ? mrow[RT - 1] : mrow[0]) : -INFINITY, mbb = lb > 0.f ? xs[64] : -INFINITY;
      const float m = fmaxf(ma, mbb);
      fa = __builtin_amdgcn_exp2f(ma - m);
      fb = __builtin_amdgcn_exp2f(mbb - m);
      inv = 1.f / (la * fa + lb * fb);
    }
#pragma unroll
    for (int t = 0; t < NTN; ++t) {
      const f32x4 ob = *reinterpret_cast<const f32x4*>(xr + t * 1024);
      const f32x4 oa = kh ? o[t][RT - 1] : o[t][0];
      oo[t] = kSoftmax ? oa * fa + ob * fb : oa + ob;
    }
  } else {
#pragma unroll
    for (int t = 0; t < NTN; ++t) oo[t] = o[t][0];
    if constexpr (kSoftmax) inv = 1.f / row_total(row_part(0));
  }

  // ---- epilogue: normalise (softmax), cast, store the wave's 16 rows: by rows through LDS where the output allows
  // (store_tile_rows), else 4 contiguous columns per lane from registers
  const bool by_rows = !p.out_f32 && (N & 7) == 0 && (p.f_rs & 7) == 0 && (p.f_bs & 7) == 0 && (p.f_bs2 & 7) == 0 &&
                       (reinterpret_cast<size_t>(p.f) & 15) == 0;  // wave-uniform
  constexpr int kRowBytes = tile_row_bytes<D>();
  constexpr int PARK = NW * XCH;  // behind the inboxes, which the other waves may still be reading
  static_assert(PARK + NW * 16 * tile_row_bytes<D>() <= NR * 2 * TB, "the parked rows need the staged tiles' LDS");
  char* const tw = smem_raw + PARK + wave * 16 * kRowBytes;
  const int m_tile = m_wave + 16 * kh;
  const int row = m_tile + c16;
  if (by_rows || row < M) {
#pragma unroll
    for (int t = 0; t < NTN; ++t) {
      const int n = 16 * t + 4 * q;
      if (!by_rows && n >= N) continue;
      float v0 = oo[t][0] * inv, v1 = oo[t][1] * inv, v2 = oo[t][2] * inv, v3 = oo[t][3] * inv;
      if (!kSoftmax && p.relu_out) { v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); v2 = fmaxf(v2, 0.f); v3 = fmaxf(v3, 0.f); }
      const long long off = zo * p.f_bs2 + zi * p.f_bs + (long long)row * p.f_rs + n;
      if (p.out_f32) {
        f32x4 w = {v0, v1, v2, v3};
        *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.f) + off) = w;
      } else {
        V2 a0 = cvt2<T>(v0, v1), a1 = cvt2<T>(v2, v3);
        V4 w = {a0[0], a0[1], a1[0], a1[1]};
        if (by_rows) *reinterpret_cast<V4*>(tw + c16 * kRowBytes + n * 2) = w;
        else *reinterpret_cast<V4*>(reinterpret_cast<T*>(p.f) + off) = w;
      }
    }
  }
  if (by_rows)
    store_tile_rows<T, D, 16>(tw, reinterpret_cast<T*>(p.f) + zo * p.f_bs2 + zi * p.f_bs + (long long)m_tile * p.f_rs,
                                    p.f_rs, M - m_tile, N, lane);
#else
  (void)p;
#endif
}

template <typename T, int D, int INTER, int KSPLIT, bool B_KL>
hipError_t launch_bmm_chain4m16(const BmmChainArgs& args, hipStream_t stream) {
  constexpr int lds = bmm_chain4m16_lds_bytes<D>();
  auto kern = bmm_chain4m16_kernel<T, D, INTER, KSPLIT, B_KL>;
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
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, args);
  return hipGetLastError();
}

}  // namespace ditto
