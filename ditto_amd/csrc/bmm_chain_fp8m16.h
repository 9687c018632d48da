// Eight-wave fused two-contraction chain on the 16x16x32 MFMA (see bmm_chain_fp.h for the chain and the
// transposed formulation, bmm_chain_fp8.h for the eight-wave workgroup and the once-per-workgroup
// transposition of the C tile into fragment-major order).
//
// Why another tile shape: on N(0,1) operands this device runs matrix code against its power limit, not
// against its clock (the same kernel on zero operands is a quarter faster), so what counts is energy per
// flop, and v_mfma_f32_16x16x32 needs about 14 % less of it than v_mfma_f32_32x32x16 (a loop of either,
// random bf16 operands, two waves per SIMD: 16.1 against 18.9 ns per 32768 flop per SIMD): it reads and
// writes a quarter of the accumulator registers per instruction.  A wave still owns 32 rows of A (two
// column tiles of 16), so every operand fragment read from LDS feeds two MFMAs and LDS traffic, register
// count and the number of direct loads are those of the 32x32x16 kernels.
//
// Layouts (lane = 16 * q + c, q = 0..3, c = 0..15):
//   v_mfma_f32_16x16x32:  A[16][32]: lane holds A[c][8q .. 8q+7];  B[32][16]: lane holds B[8q .. 8q+7][c];
//                         acc[r] = C[4q + r][c], r = 0..3.
//   first contraction, transposed:  S^T[l][m] = sum_k B^T[l][k] A^T[k][m]
//       A operand  = 16 rows l of the B tile (stored [L][K]: one 16-byte read per lane),
//       B operand  = rows m of A from registers (lane: row 16j + c, 8 consecutive k),
//       result     = lane (c, q) holds S^T[16i + 4q + r][16j + c]: four consecutive l of row m.
//   second contraction, transposed:  F^T[n][m] = sum_l C^T[n][l] P^T[l][m] over the 32 rows of a half tile
//       B operand  = P^T from the accumulators above: slot e < 4 is row 4q + e of the first 16-row tile,
//                    slot e >= 4 row 4q + e - 4 of the second, i.e. contraction slot 8q + e <-> row
//                    pi(8q + e) = 4q + e (e < 4), 16 + 4q + e - 4 (e >= 4);
//       A operand  = C^T with its rows taken in the same order pi: lane (n = c, q) holds
//                    C[pi(8q + e)][16t + c], e = 0..7: two transposing reads of 4 rows x 16 columns, done once
//                    per workgroup by the wave that owns the fragment and written back fragment major.
//
// Softmax: a lane holds eight scores of each of two rows per half tile.  The running maximum of a row is
// shared by its four lanes and raised lazily; whether it has to be raised is decided from the lanes' LOCAL
// maxima (a ballot), so the usual case needs no exchange between lanes at all; the exchange
// (v_permlane16_swap, v_permlane32_swap) runs only in the rare rescale.
#pragma once
#include "bmm_chain_fp8.h"

namespace ditto {

template <int D>
__host__ __device__ constexpr int bmm_chain8m16_lds_bytes() {
  // B tiles as loaded [4], raw C tiles [4], fragment-major C tiles [2]
  return (4 + 4 + 2) * kBN * D * 2;
}

template <typename V8>
struct ElemOf;
template <>
struct ElemOf<f16x8> {
  typedef f16 type;
};
template <>
struct ElemOf<bf16x8> {
  typedef bf16 type;
};

template <typename T>
struct Mfma16;
template <>
struct Mfma16<f16> {
  static __device__ __forceinline__ f32x4 run(f16x8 a, f16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mfma16<bf16> {
  static __device__ __forceinline__ f32x4 run(bf16x8 a, bf16x8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};

// The output accumulators live in FIXED registers, v[4 i : 4 i + 3] for accumulator i: every statement that
// writes one is followed by an empty asm that names that register as a tied operand.  Left to itself the
// compiler gives an MFMA's result another register than the accumulator came in (it likes to reuse the first
// operand's) and computes the rare rescale into fresh registers, so the accumulators change places and the
// common path of every branch copies all 64 of them back, every half step.  With source and result pinned to
// the same register the MFMA is allocated in place.  The MFMAs themselves stay the compiler's own
// instructions, so that it keeps its hazard bookkeeping: whatever reads an accumulator next (the rescale, the
// epilogue, a copy the register allocator decides on) waits for the matrix pipeline as far as it must.
__device__ __forceinline__ void acc_pin(int i, f32x4& x) {
  switch (i) {
    case 0: asm volatile("" : "+{v[0:3]}"(x)); break;
    case 1: asm volatile("" : "+{v[4:7]}"(x)); break;
    case 2: asm volatile("" : "+{v[8:11]}"(x)); break;
    case 3: asm volatile("" : "+{v[12:15]}"(x)); break;
    case 4: asm volatile("" : "+{v[16:19]}"(x)); break;
    case 5: asm volatile("" : "+{v[20:23]}"(x)); break;
    case 6: asm volatile("" : "+{v[24:27]}"(x)); break;
    case 7: asm volatile("" : "+{v[28:31]}"(x)); break;
    case 8: asm volatile("" : "+{v[32:35]}"(x)); break;
    case 9: asm volatile("" : "+{v[36:39]}"(x)); break;
    case 10: asm volatile("" : "+{v[40:43]}"(x)); break;
    case 11: asm volatile("" : "+{v[44:47]}"(x)); break;
    case 12: asm volatile("" : "+{v[48:51]}"(x)); break;
    case 13: asm volatile("" : "+{v[52:55]}"(x)); break;
    case 14: asm volatile("" : "+{v[56:59]}"(x)); break;
    case 15: asm volatile("" : "+{v[60:63]}"(x)); break;
    case 16: asm volatile("" : "+{v[64:67]}"(x)); break;
    case 17: asm volatile("" : "+{v[68:71]}"(x)); break;
    case 18: asm volatile("" : "+{v[72:75]}"(x)); break;
    case 19: asm volatile("" : "+{v[76:79]}"(x)); break;
    case 20: asm volatile("" : "+{v[80:83]}"(x)); break;
    case 21: asm volatile("" : "+{v[84:87]}"(x)); break;
    case 22: asm volatile("" : "+{v[88:91]}"(x)); break;
    case 23: asm volatile("" : "+{v[92:95]}"(x)); break;
  }
}
constexpr int kMaxAcc = 24;
template <typename V8>
__device__ __forceinline__ void acc_mfma(int i, V8 a, V8 b, f32x4 (&o)[kMaxAcc]) {
  o[i] = Mfma16<typename ElemOf<V8>::type>::run(a, b, o[i]);
  acc_pin(i, o[i]);
}
__device__ __forceinline__ void acc_scale(int i, float alpha, f32x4 (&o)[kMaxAcc]) {
  o[i] *= alpha;
  acc_pin(i, o[i]);
}

// maximum over the four lanes c, c + 16, c + 32, c + 48 (every lane gets it).
// v_permlane16_swap a, b swaps the odd rows of 16 lanes of a with the even rows of b; from a == b == x,
// max(a, b) holds max(x[row 0], x[row 1]) in rows 0 and 1 and max(x[row 2], x[row 3]) in rows 2 and 3.
__device__ __forceinline__ float quad_max(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return pair_max(fmaxf(a, b));
}
__device__ __forceinline__ float quad_sum(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
  return pair_sum(a + b);
}

// XOR applied to the 16-byte chunk index of a 128-byte row ([k][64 l] tiles of a B stored [K][L]) for the
// transposing read with lanes (c, q) -> row 4 q + c / 4: 2.3 cycles per instruction with eight waves reading, against
// 4 under the swizzle of the once-per-tile transposition passes
__device__ __forceinline__ int swz_kl_tr(int row) { return 2 * ((row >> 1) & 3); }

// The lane's id within its wave, computed where it is called (from an asm the compiler neither hoists nor merges):
// for code behind a long loop that would otherwise keep the id in a register through it.
__device__ __forceinline__ int fresh_lane_id() {
  int ln;
  asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
  return ln;
}

template <bool B>
struct BoolC {
  static constexpr bool value = B;
};
// a lane's partial row sum above which the optimistic walk lowers the row's scale (2^32)
constexpr float kSumLimitBf16 = 4294967296.f;
// fp16: a probability overflows at 2^16, so the scale is lowered from 2^8 on and a row whose scores climb by more
// than 2^8 within one tile of 64 keys ends with an infinite sum (and takes the exact walk)
constexpr float kSumLimitF16 = 256.f;

// One workgroup's walk: eight waves of RT 16-row tiles each, rows row0 .. row0 + 128 RT - 1 of batch entry bz.
template <typename T, int D, int INTER, int RT, bool B_KL>
__device__ __forceinline__ void bmm_chain8m16_body(const BmmChainArgs& p, char* smem_raw, int row0, int bz) {
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  typedef typename Elem<T>::v2 V2;
  constexpr int NW = 8;
#ifdef DITTO_M16_NO_OPTIMISTIC
  constexpr bool kOptimistic = false;
#else
  constexpr bool kOptimistic = INTER == kInterSoftmax;
#endif
  constexpr float kSumLimit = Elem<T>::is_bf16 ? kSumLimitBf16 : kSumLimitF16;
  constexpr int TB = kBN * D * 2;     // bytes per tile
  // bytes per LDS row of a B tile: [L][K] as stored, or, with B stored [K][L], [K][64 l]
  constexpr int B_RB = B_KL ? kBN * 2 : D * 2;
  constexpr int B_CPR = B_RB / 16;
  constexpr int C_RB = D * 2;
  constexpr int C_CPR = C_RB / 16;
  constexpr int NS = D / 32;          // k steps of the first contraction
  constexpr int NTN = D / 16;         // column tiles of the second contraction
  constexpr int NFRAG = 2 * NTN;      // C fragments per tile: two 32-row halves x NTN column tiles
  constexpr int NLD = TB / 1024 / NW; // direct loads per wave per tile
  constexpr int NTR = NFRAG / NW;     // fragments each wave transposes per tile
  static_assert(NLD >= 1 && NTR >= 1, "tile too small for eight waves");
  constexpr int NCR = 4;
  constexpr int B_LOAD = 0;                   // [4] row-read layout
  constexpr int C_RAW = 4 * TB;               // [NCR]
  constexpr int C_FRAG = C_RAW + NCR * TB;    // [2]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15, q = lane >> 4;
  // A half step has a phase that is heavy on the vector ALU (first contraction of the coming half tile, with
  // the exponentials of the current one between its MFMAs) and one that is MFMAs only (second contraction of
  // the current one).  Taking the phases in the other order changes nothing measurable, and letting the two
  // waves of a SIMD take different orders, so that one wave's exponentials meet the other's MFMAs, is slower
  // (506 against 437 us at 64 x 4096 x 4096 x 128 on zero operands): what limits a half step is the register
  // file's write port, which the fragments returning from LDS (four registers per 16-byte read), the vector
  // ALU's results and the MFMAs share.  A loop of two 16x16x32 MFMAs, one ds_read_b128 and n vector
  // instructions per wave, two waves per SIMD, takes 39, 55 and 60 cycles for n = 0, 4, 6 (34, 36 and 43
  // without the read; 32 is the matrix pipe's own time): about four register writes per MFMA pair are free,
  // each further one costs four cycles.  This kernel has the read and about 5.6 vector results per pair.

  const int zo = bz / p.batch_inner, zi = bz - zo * p.batch_inner;
  const T* __restrict__ Ag = reinterpret_cast<const T*>(p.a) + zo * p.a_bs2 + zi * p.a_bs;
  const T* Bg = reinterpret_cast<const T*>(p.b) + zo * p.b_bs2 + zi * p.b_bs;
  const T* Cg = reinterpret_cast<const T*>(p.c) + zo * p.c_bs2 + zi * p.c_bs;
  const int m_wave = row0 + wave * 16 * RT;
  const int M = p.M, N = p.N, K = p.K, L = p.L;

  const unsigned b_bytes = (unsigned)(B_KL ? ((long long)(K - 1) * p.b_rs + L) : ((long long)(L - 1) * p.b_rs + K)) * 2u;
  const unsigned c_bytes = (unsigned)((long long)(L - 1) * p.c_rs + N) * 2u;
  const i32x4 b_rsrc = make_rsrc(Bg, b_bytes);
  const i32x4 c_rsrc = make_rsrc(Cg, c_bytes);
  const unsigned lds0 = (unsigned)(size_t)(DITTO_LDS char*)smem_raw;

  // ---- per-lane source offsets of the direct loads (the swizzles of the other kernels)
  int b_voff[NLD], c_voff[NLD];
#pragma unroll
  for (int i = 0; i < NLD; ++i) {
    const int gi = NLD * wave + i;
    {
      const int row = gi * (64 / B_CPR) + lane / B_CPR, pc = lane % B_CPR;
      if (B_KL) {
        const int cl = pc ^ swz_kl_tr(row);  // rows are k, columns l
        b_voff[i] = row < K ? (row * p.b_rs + cl * 8) * 2 : (int)b_bytes;
      } else {
        const int cl = pc ^ swz_rowread<B_CPR>(row);  // rows are l, columns k
        b_voff[i] = cl * 8 < K ? (row * p.b_rs + cl * 8) * 2 : (int)b_bytes;
      }
    }
    {
      const int row = gi * (64 / C_CPR) + lane / C_CPR, pc = lane % C_CPR;
      const int cl = pc ^ swz_trread<C_CPR>(row);
      c_voff[i] = cl * 8 < N ? (row * p.c_rs + cl * 8) * 2 : (int)c_bytes;
    }
  }
  auto load_b = [&](int tile, int buf) __attribute__((always_inline)) {
    int soff = B_KL ? tile * kBN * 2 : tile * kBN * p.b_rs * 2;
    asm volatile("" : "+s"(soff));  // one add per load, not a hoisted address register per load and tile slot
    // B stored [K][L]: the first column l (within the tile) the lane loads is the same for all of its loads (their rows
    // differ by multiples of 8 and the swizzle looks at row % 8: lane / 8 here); taken from the lane id afresh rather
    // than kept in a register through the walk
    int b_col = 0;
    if (B_KL) {
      const int ln = fresh_lane_id();
      b_col = 8 * ((ln & 7) ^ swz_kl_tr(ln >> 3));
    }
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      int vo = b_voff[i] + soff;
      if (B_KL) vo = (tile * kBN + b_col < L) ? vo : (int)b_bytes;  // columns past L lie inside the buffer (the next row)
      lds_dma_16(b_rsrc, (unsigned)vo, lds0 + B_LOAD + buf * TB + 1024 * (NLD * wave + i));
    }
  };
  auto load_c = [&](int tile, int buf) __attribute__((always_inline)) {
    int soff = tile * kBN * p.c_rs * 2;
    asm volatile("" : "+s"(soff));
#pragma unroll
    for (int i = 0; i < NLD; ++i)
      lds_dma_16(c_rsrc, (unsigned)(c_voff[i] + soff), lds0 + C_RAW + buf * TB + 1024 * (NLD * wave + i));
  };

  // ---- per-lane LDS read addresses (bytes within a tile), loop invariant
  // B fragment (i = 16-row tile of the 64-row L tile, st = k step): row 16 i + c, logical chunks 4 st + q
  // (256-byte rows: the swizzle of row 16 i + c does not depend on i, so the tile index is a constant offset)
  // B stored [K][L]: the tile is [k][64 l], 128-byte rows, and fragment (i, st) comes out of two transposing reads
  // like a C fragment does in the transposition pass: rows 32 st + 4 q + {0..3} (and + 16) x columns 16 i .. + 15,
  // so its contraction index runs 4 q .. + 3, 16 + 4 q .. + 3 within the step and the A fragments are loaded in
  // that order; the address depends on i (the swizzle on the row % 8 only), the k step is a constant offset
  constexpr int NBI = B_KL ? 4 : B_CPR == 16 ? 1 : 4;
  constexpr int NBS = B_KL ? 1 : NS;
  int b_ad[NBI][NBS];
  if (B_KL) {
#pragma unroll
    for (int i = 0; i < NBI; ++i) {
      const int row = 4 * q + (c16 >> 2);
      const int chunk = 2 * i + ((c16 & 3) >> 1);
      b_ad[i][0] = row * B_RB + ((chunk ^ swz_kl_tr(row)) * 16) + 8 * (c16 & 1);
    }
  } else {
#pragma unroll
    for (int i = 0; i < NBI; ++i)
#pragma unroll
      for (int st = 0; st < NBS; ++st)
        b_ad[i][st] = (16 * i + c16) * B_RB + (((4 * st + q) ^ swz_rowread<B_CPR>(16 * i + c16)) * 16);
  }
  // Fragment-major and raw C tiles lie beyond the 64 KB an LDS instruction's offset field reaches: each
  // region gets ONE base register, kept opaque so that the compiler folds only the small remainder into the
  // instructions' offsets (it otherwise makes an address register per buffer and fragment, and spills)
  int frag_ad = lane * 16 + C_FRAG;
  asm volatile("" : "+v"(frag_ad));
  auto b_frag = [&](int off, int i, int st) __attribute__((always_inline)) -> V8 {
    if (B_KL) {
      const char* a = smem_raw + b_ad[i % NBI][0] + (off + 32 * st * B_RB);
      V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(a));
      V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(a + 16 * B_RB));
      return concat4<V4, V8>(lo, hi);
    }
    if (NBI == 1) return *reinterpret_cast<const V8*>(smem_raw + b_ad[0][st % NBS] + (off + 16 * i * B_RB));
    return *reinterpret_cast<const V8*>(smem_raw + b_ad[i % NBI][st % NBS] + off);
  };
  auto frag_rd = [&](int off, int f) __attribute__((always_inline)) -> V8 {
    return *reinterpret_cast<const V8*>(smem_raw + frag_ad + (off - C_FRAG + 1024 * f));
  };
  // This wave's share of the transposition of one C tile: fragments NTR * wave .. + NTR - 1, fragment
  // f = hh * NTN + t (hh: 32-row half, t: 16-column tile).  The 16 lanes of group q read rows
  // 32 hh + 4 q + {0..3} (and + 16) x columns 16 t .. 16 t + 15: lane s of the group points at row s / 4,
  // 8 bytes at column 4 (s % 4).
  int ctr_ad[NTR], fw_ad[NTR];
#pragma unroll
  for (int i = 0; i < NTR; ++i) {
    const int f = NTR * wave + i;
    const int hh = f / NTN, t = f % NTN;
    const int row = 32 * hh + 4 * q + (c16 >> 2);
    const int chunk = 2 * t + ((c16 & 3) >> 1);
    // (rows row and row + 16 share their swizzle: it depends on row % 4 only)
    ctr_ad[i] = row * C_RB + ((chunk ^ swz_trread<C_CPR>(row)) * 16) + 8 * (c16 & 1) + C_RAW;
    fw_ad[i] = frag_ad + 1024 * f;
    asm volatile("" : "+v"(ctr_ad[i]), "+v"(fw_ad[i]));
  }
  auto tr_read_c = [&](int raw_off, V8* x) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NTR; ++i) {
      const char* a = smem_raw + ctr_ad[i] + (raw_off - C_RAW);
      V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(a));
      V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(a + 16 * C_RB));
      x[i] = concat4<V4, V8>(lo, hi);
    }
  };
  auto tr_write = [&](int frag_off, const V8* x) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NTR; ++i) *reinterpret_cast<V8*>(smem_raw + fw_ad[i] + (frag_off - C_FRAG)) = x[i];
  };

  // ---- A fragments (B operand of the first contraction): lane holds A[16 j + c][32 st + 8 q .. + 7]
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

  // ---- accumulators of F^T: o[t][j][r] = F^T[16 t + 4 q + r][16 j + c]
  // (flat: accumulator RT t + j, pinned to v[4 (RT t + j) : +3], see acc_mfma)
  static_assert(RT * NTN <= kMaxAcc, "pinned accumulators");
  f32x4 o[kMaxAcc];
#pragma unroll
  for (int i = 0; i < RT * NTN; ++i) o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  // softmax state of the lane's two rows: running maximum (exp2 domain; the same in the four lanes of a
  // row), the lane's share of the row sum, and the lane's LOCAL scaled maximum of the half about to be consumed
  float mrow[RT], lsum[RT], mloc[RT];
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    mrow[j] = -INFINITY;
    lsum[j] = 0.f;
    mloc[j] = -INFINITY;
  }
  const float c2 = p.scale_log2;
  const int ntiles = (L + kBN - 1) / kBN;
  const bool ragged = (L % kBN) != 0;

  // A half tile of scores: sc[i][j] = 16-row tile i x row tile j
  struct Half {
    f32x4 v[2][RT];
  };
  Half sa, sb;
  auto mask_tail = [&](Half& h, int l0) __attribute__((always_inline)) {
    const int rem = L - l0 - 4 * q;  // rows left, counted from the lane's first (compared with constants below)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int gone = (rem - (16 * i + r) - 1) >> 31;  // all ones where 16 i + r >= rem
#pragma unroll
        for (int j = 0; j < RT; ++j) h.v[i][j][r] = neg_inf_where(h.v[i][j][r], gone);
      }
  };
  auto local_max = [&](const Half& h) __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < RT; ++j) {
      float mx = h.v[0][j][0];
#pragma unroll
      for (int r = 1; r < 4; ++r) mx = fmaxf(mx, h.v[0][j][r]);
#pragma unroll
      for (int r = 0; r < 4; ++r) mx = fmaxf(mx, h.v[1][j][r]);
      mloc[j] = mx * c2;
    }
  };
  // probabilities of 16-row tile i of the half, row tile j: unit u = 0 .. 2 RT - 1 is (i = u / RT, j = u % RT)
  auto exp_unit = [&](Half& h, int u) __attribute__((always_inline)) {
    const int i = u / RT, j = u % RT;
#pragma unroll
    for (int r = 0; r < 4; ++r) h.v[i][j][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(h.v[i][j][r], c2, -mrow[j]));
    // keep the unit where it is called, between the MFMAs of its group: statements with side effects keep
    // their order, plain arithmetic is otherwise free to sink to its use
    asm volatile("" : "+v"(h.v[i][j][0]), "+v"(h.v[i][j][1]), "+v"(h.v[i][j][2]), "+v"(h.v[i][j][3]));
  };
  // operand of the second contraction for row tile j: slots 0..3 from the first 16-row tile, 4..7 from the
  // second; the row sum is taken over the ROUNDED values, exactly what enters the MFMA
  auto make_p = [&](const Half& h, int j, V8& pf) __attribute__((always_inline)) {
    float v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[e] = h.v[e >> 2][j][e & 3];
      if (INTER != kInterSoftmax && p.relu) v[e] = fmaxf(v[e], 0.f);
    }
    V2 p0 = cvt2<T>(v[0], v[1]), p1 = cvt2<T>(v[2], v[3]), p2 = cvt2<T>(v[4], v[5]), p3 = cvt2<T>(v[6], v[7]);
    if constexpr (INTER == kInterSoftmax) {
      lsum[j] = Elem<T>::add_pair(p0, lsum[j]);
      lsum[j] = Elem<T>::add_pair(p1, lsum[j]);
      lsum[j] = Elem<T>::add_pair(p2, lsum[j]);
      lsum[j] = Elem<T>::add_pair(p3, lsum[j]);
    }
    pf = V8{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  };
  // Lazy rescale, decided without any exchange between lanes: a lane votes when its local maximum exceeds the
  // row's running maximum by more than 2^kLazy.  Only then are the row maxima exchanged (all rows of the
  // wave: a raised maximum must be the same in the four lanes of its row) and the accumulators rescaled.
  auto maybe_rescale = [&]() __attribute__((always_inline)) {
    bool vote = false;
#pragma unroll
    for (int j = 0; j < RT; ++j) vote = vote || mloc[j] > mrow[j] + kLazy;
    if (__builtin_amdgcn_ballot_w64(vote) != 0) {
#pragma unroll
      for (int j = 0; j < RT; ++j) {
        const float mnew = fmaxf(mrow[j], quad_max(mloc[j]));
        const float alpha = __builtin_amdgcn_exp2f(mrow[j] - mnew);  // (-inf) - (-inf) does not occur: mnew is finite
        mrow[j] = mnew;
        lsum[j] *= alpha;
#pragma unroll
        for (int t = 0; t < NTN; ++t) acc_scale(RT * t + j, alpha, o);
      }
    }
  };

  // The optimistic walk (bf16): no maximum is taken per half tile.  The row's reference exponent is the maximum of
  // its first 32 scores, and what is watched is the row SUM: a probability is never larger than the sum it went
  // into, so while a lane's partial sum stays below 2^kSumLimitLog2 no probability has come near the end of the
  // fp32 / bf16 range.  Once per tile a lane votes when its sum has passed the limit; the row's reference is then
  // raised by a whole number of binary orders (scaling by a power of two is exact) and sums and accumulators follow.
  // A row whose scores climb by more than the range within one tile overflows before the vote: its sum ends up
  // infinite or NaN, which the end of the walk detects, and the workgroup then walks the keys again the exact way
  // (maximum per half tile before any exponential).
  auto sum_rescale = [&]() __attribute__((always_inline)) {
    float smax = lsum[0];
#pragma unroll
    for (int j = 1; j < RT; ++j) smax = fmaxf(smax, lsum[j]);
    if (__builtin_amdgcn_ballot_w64(smax > kSumLimit) != 0) {
#pragma unroll
      for (int j = 0; j < RT; ++j) {
        const float sref = quad_max(lsum[j]);  // the same in the four lanes of a row
        // (an infinite or NaN sum is left as it is: that is what the end of the walk looks for)
        const int e = (sref > kSumLimit && sref < INFINITY) ? ((__builtin_bit_cast(int, sref) >> 23) & 255) - 127 : 0;
        const float alpha = __builtin_bit_cast(float, (127 - e) << 23);  // 2^-e, 32 <= e <= 127
        mrow[j] += (float)e;
        lsum[j] *= alpha;
#pragma unroll
        for (int t = 0; t < NTN; ++t) acc_scale(RT * t + j, alpha, o);
      }
    }
  };
  // reference exponent of a fresh row: the maximum of its first half tile (finite: key 0 exists and is not masked)
  auto init_max = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int j = 0; j < RT; ++j) mrow[j] = quad_max(mloc[j]);
  };

  // One half step: consumes `cur` (half hh of tile it), produces `nxt` (the following half).  Fragment
  // groups: 2 NS of the first contraction (16-row tile i of the next half x k step), then NTN of the second
  // (column tile t); each fragment feeds the two row tiles.
  // fragments in flight ahead of the MFMAs: 4 measured best on the 64 x 4096 x 4096 x 128 attention (2: +0.5 %, 6: +0.3 %,
  // 8: +10 %, the registers run out)
  constexpr int kAhead = 4;
  constexpr int NGS = 2 * NS, NG = NGS + NTN;
  auto half_step = [&](Half& cur, Half& nxt, int it, auto j_c, auto hh_c, auto safe_c) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value, hh = decltype(hh_c)::value;
    constexpr bool SAFE = decltype(safe_c)::value;
    constexpr int BNX = B_LOAD + (hh ? (J + 1) % 4 : J) * TB;  // B tile of the next half
    constexpr int CF = C_FRAG + (J & 1) * TB;
    if constexpr (INTER == kInterSoftmax && SAFE) maybe_rescale();
    V8 fr[NG];
    auto fetch = [&](int k) __attribute__((always_inline)) {
      // first contraction: k = st * 2 + i (the two 16-row tiles of the half alternate: four accumulators in turn)
      fr[k] = k < NGS ? b_frag(BNX, 2 * (hh ^ 1) + (k & 1), k >> 1) : frag_rd(CF, hh * NTN + (k - NGS));
    };
#pragma unroll
    for (int k = 0; k < kAhead; ++k) fetch(k);
    V8 pf[RT];
    // vector phase first, all of it, then the MFMAs of both contractions back to back
    auto vphase = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (INTER == kInterSoftmax) {
#pragma unroll
      for (int u = 0; u < 2 * RT; ++u) exp_unit(cur, u);
    }
#pragma unroll
    for (int j = 0; j < RT; ++j) {
      make_p(cur, j, pf[j]);
      // (the row sum is named too: left free, its dots sink to the end of the tile, and the rounded pairs they read
      // then have to be kept in a second set of registers next to the operand)
      asm volatile("" : "+v"(pf[j]), "+v"(lsum[j]));
    }
    __builtin_amdgcn_sched_barrier(0);
    };
    vphase();
#pragma unroll
    for (int k = 0; k < NG; ++k) {
      if (k + kAhead < NG) fetch(k + kAhead);
      __builtin_amdgcn_sched_barrier(0);
      if (k < NGS) {
        const int i = k & 1, st = k >> 1;
#pragma unroll
        for (int j = 0; j < RT; ++j) {
          if (st == 0) nxt.v[i][j] = Mfma16<T>::run(fr[k], af[j][st], f32x4{0.f, 0.f, 0.f, 0.f});
          else nxt.v[i][j] = Mfma16<T>::run(fr[k], af[j][st], nxt.v[i][j]);
        }
      } else {
        const int t = k - NGS;
#pragma unroll
        for (int j = 0; j < RT; ++j) acc_mfma(RT * t + j, fr[k], pf[j], o);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (INTER == kInterSoftmax) {
      const int nt = hh ? it + 1 : it;  // tile of the next half
      if (ragged && nt == ntiles - 1) mask_tail(nxt, nt * kBN + 32 * (hh ^ 1));
      if constexpr (SAFE) local_max(nxt);
    }
  };
  auto tile_step = [&](int it, auto j_c, auto safe_c) __attribute__((always_inline)) {
    constexpr int J = decltype(j_c)::value;
    constexpr bool SAFE = decltype(safe_c)::value;
    constexpr int PAR = J & 1;
    V8 xc[NTR];
    tr_read_c(C_RAW + ((J + 1) % 4) * TB, xc);
    half_step(sa, sb, it, j_c, IntC<0>{}, safe_c);
    tr_write(C_FRAG + (PAR ^ 1) * TB, xc);
    half_step(sb, sa, it, j_c, IntC<1>{}, safe_c);
    if constexpr (INTER == kInterSoftmax && !SAFE) sum_rescale();
    // The direct loads of tile it + 3 go out here, at the END of the step, into the slot of tile it - 1 (last read
    // before the previous barrier): a wave whose loads queue up behind the workgroup's others then waits where it
    // would wait for the barrier anyway, and the waves reach this point at different times.  Issued behind the
    // barrier, all at once, the same loads held every wave up at the start of its step (2 % of the launch).
    // What must have landed before the barrier is tile it + 2 (transposed from the next step's first instruction
    // on); the 2 NLD loads just issued may stay in flight.
    load_c(it + 3, (J + 3) % 4);
    load_b(it + 3, (J + 3) % 4);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NLD) : "memory");
    __syncthreads();
  };

  // ---- one walk over the keys: prologue (first tiles in flight, first transposition, scores of the very first
  // half), then the tile loop
  auto walk = [&](auto safe_c) __attribute__((always_inline)) {
  constexpr bool SAFE = decltype(safe_c)::value;
  load_b(0, 0);
  load_b(1, 1);
  load_c(0, 0);
  load_c(1, 1);
  load_b(2, 2);
  load_c(2, 2);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  {
    V8 x[NTR];
    tr_read_c(C_RAW, x);
    tr_write(C_FRAG, x);
  }
#pragma unroll
  for (int st = 0; st < NS; ++st)
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const V8 bf = b_frag(B_LOAD, i, st);
#pragma unroll
      for (int j = 0; j < RT; ++j) {
        if (st == 0) sa.v[i][j] = Mfma16<T>::run(bf, af[j][st], f32x4{0.f, 0.f, 0.f, 0.f});
        else sa.v[i][j] = Mfma16<T>::run(bf, af[j][st], sa.v[i][j]);
      }
    }
  if constexpr (INTER == kInterSoftmax) {
    if (ragged && ntiles == 1) mask_tail(sa, 0);
    local_max(sa);
    if constexpr (!SAFE) init_max();
  }
  __syncthreads();

  for (int it = 0; it < ntiles; it += 4) {
    tile_step(it, IntC<0>{}, safe_c);
    if (it + 1 < ntiles) tile_step(it + 1, IntC<1>{}, safe_c);
    if (it + 2 < ntiles) tile_step(it + 2, IntC<2>{}, safe_c);
    if (it + 3 < ntiles) tile_step(it + 3, IntC<3>{}, safe_c);
  }
  };  // walk

  if constexpr (kOptimistic) {
    walk(BoolC<false>{});
    // a sum that is not finite (or NaN) in any lane of the workgroup sends all of it through the exact walk:
    // the tiles are a workgroup's common property.  The flag lives in the fragment-major region, which no direct
    // load writes; loads of tiles past the last one may still be landing elsewhere.
    bool bad = false;
#pragma unroll
    for (int j = 0; j < RT; ++j) bad = bad || !(lsum[j] < INFINITY);
    int* const flag = reinterpret_cast<int*>(smem_raw);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no direct load still on its way into LDS
    wg_sync();
    // (B stored [K][L]: that instantiation has no register left to keep the lane id through the walk)
    const int lane_f = B_KL ? fresh_lane_id() : lane;
    if (B_KL ? (lane_f == 0 && wave == 0) : tid == 0) *flag = 0;
    wg_sync();
    if (__builtin_amdgcn_ballot_w64(bad) != 0 && lane_f == 0) *flag = 1;
    wg_sync();
    const int again = __builtin_amdgcn_readfirstlane(*flag);
    if (again) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      wg_sync();
#pragma unroll
      for (int i = 0; i < RT * NTN; ++i) {
        o[i] = f32x4{0.f, 0.f, 0.f, 0.f};
        acc_pin(i, o[i]);
      }
#pragma unroll
      for (int j = 0; j < RT; ++j) {
        mrow[j] = -INFINITY;
        lsum[j] = 0.f;
        mloc[j] = -INFINITY;
      }
      walk(BoolC<true>{});
    }
  } else {
    walk(BoolC<true>{});
  }

  // ---- epilogue: normalise (softmax), cast, store: by rows through LDS (free by now) where the output allows
  // (store_tile_rows), else 4 contiguous columns per lane from registers
  const bool by_rows = !p.out_f32 && (N & 7) == 0 && (p.f_rs & 7) == 0 && (p.f_bs & 7) == 0 && (p.f_bs2 & 7) == 0 &&
                       (reinterpret_cast<size_t>(p.f) & 15) == 0;  // wave-uniform
  constexpr int kRowBytes = tile_row_bytes<D>();
  static_assert(8 * (16 * RT) * tile_row_bytes<D>() <= bmm_chain8m16_lds_bytes<D>(), "the parked rows need the staged tiles' LDS");
  if (by_rows) {
    // every wave is done with the staged tiles, and the direct loads still in flight (the tiles past the last one:
    // zeros) have landed -- they would otherwise fall on the rows parked below
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    wg_sync();
  }
  char* const tw = smem_raw + wave * 16 * RT * kRowBytes;
  // lane coordinates taken afresh: values kept from the prologue for this would sit in registers (or spill)
  // through the whole walk
  int lane_e = threadIdx.x & 63;
  asm volatile("" : "+v"(lane_e));
  const int c16e = lane_e & 15, qe = lane_e >> 4;
#pragma unroll
  for (int j = 0; j < RT; ++j) {
    float inv = 1.f;
    if constexpr (INTER == kInterSoftmax) inv = 1.f / quad_sum(lsum[j]);
    const int row = m_wave + 16 * j + c16e;
    if (!by_rows && row >= M) continue;
#pragma unroll
    for (int t = 0; t < NTN; ++t) {
      const int n = 16 * t + 4 * qe;
      if (!by_rows && n >= N) continue;
      float v0 = o[RT * t + j][0] * inv, v1 = o[RT * t + j][1] * inv, v2 = o[RT * t + j][2] * inv, v3 = o[RT * t + j][3] * inv;
      if (INTER != kInterSoftmax && p.relu_out) { v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); v2 = fmaxf(v2, 0.f); v3 = fmaxf(v3, 0.f); }
      const long long off = zo * p.f_bs2 + zi * p.f_bs + (long long)row * p.f_rs + n;
      if (p.out_f32) {
        f32x4 w = {v0, v1, v2, v3};
        *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.f) + off) = w;
      } else {
        V2 a0 = cvt2<T>(v0, v1), a1 = cvt2<T>(v2, v3);
        V4 w = {a0[0], a0[1], a1[0], a1[1]};
        if (by_rows) *reinterpret_cast<V4*>(tw + (16 * j + c16e) * kRowBytes + n * 2) = w;
        else *reinterpret_cast<V4*>(reinterpret_cast<T*>(p.f) + off) = w;
      }
    }
  }
  if (by_rows)
    store_tile_rows<T, D, 16 * RT>(tw, reinterpret_cast<T*>(p.f) + zo * p.f_bs2 + zi * p.f_bs + (long long)m_wave * p.f_rs, p.f_rs,
                              M - m_wave, N, lane_e);
}

// Workgroups come in two sizes: the first p.mblocks3 row blocks of a batch entry have 384 rows (three 16-row tiles
// per wave: an operand fragment read from LDS feeds three MFMAs, and the per-tile overheads - direct loads,
// transposition, barrier - are spread over half as many MFMAs again), the others 256.  The split lets a row count
// that 384 does not divide fill the device evenly: 4096 rows on four compute units are 2 x 384 + 256 each.  Ids are
// dealt so that every XCD first gets the large blocks of all of its batch entries, then the small ones (longest
// first: the small blocks fill the gaps at the end).
template <typename T, int D, int INTER, bool B_KL>
__global__ __launch_bounds__(512) void bmm_chain8m16_kernel(BmmChainArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  const int nb3 = p.mblocks3, nb2 = p.mblocks - p.mblocks3;
  int x = 0, idx = blockIdx.x, per = p.batch;  // XCD, position in the XCD's dispatch order, batch entries per XCD
  if (gridDim.x % 8 == 0 && p.batch % 8 == 0) {
    x = blockIdx.x & 7;
    idx = blockIdx.x >> 3;
    per = p.batch >> 3;
  }
  if (idx < per * nb3) {
    const int e = idx / nb3, mb = idx - e * nb3;
    bmm_chain8m16_body<T, D, INTER, 3, B_KL>(p, smem_raw, 384 * mb, x * per + e);
  } else {
    const int r = idx - per * nb3;
    const int e = r / nb2, mb = r - e * nb2;
    bmm_chain8m16_body<T, D, INTER, 2, B_KL>(p, smem_raw, 384 * nb3 + 256 * mb, x * per + e);
  }
#else
  (void)p;
#endif
}

template <typename T, int D, int INTER, bool B_KL>
hipError_t launch_bmm_chain8m16(const BmmChainArgs& args, hipStream_t stream) {
  constexpr int lds = bmm_chain8m16_lds_bytes<D>();
  auto kern = bmm_chain8m16_kernel<T, D, INTER, B_KL>;
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
