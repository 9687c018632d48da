// Shared device/host helpers for the gfx950 chain kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ditto {

typedef _Float16 f16;
typedef __bf16 bf16;

typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(2))) int i32x2;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(2))) unsigned u32x2;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

#define DITTO_LDS __attribute__((address_space(3)))

// Per-element-type traits: vector types and the gfx950 MFMA that consumes them.
//   32x32x16: A lane l holds A[l%32][8*(l/32)+0..7], B lane l holds B[8*(l/32)+0..7][l%32],
//             acc[r] = C[8*(r/4) + 4*(l/32) + r%4][l%32].
template <typename T>
struct Elem;

template <>
struct Elem<f16> {
  static constexpr bool is_bf16 = false;
  typedef f16x8 v8;
  typedef f16x4 v4;
  typedef f16x2 v2;
  static __device__ __forceinline__ f32x16 mfma32(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(v8 a, v8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  // acc + p[0] + p[1] in one instruction (v_dot2c_f32_f16 against a pair of ones)
  static __device__ __forceinline__ float add_pair(v2 p, float acc) {
    const v2 ones = {(f16)1.0f, (f16)1.0f};
    return __builtin_amdgcn_fdot2(p, ones, acc, false);
  }
  // acc + a[0]*b[0] + a[1]*b[1] in fp32 (v_dot2_f32_f16)
  static __device__ __forceinline__ float dot2(v2 a, v2 b, float acc) { return __builtin_amdgcn_fdot2(a, b, acc, false); }
};

template <>
struct Elem<bf16> {
  static constexpr bool is_bf16 = true;
  typedef bf16x8 v8;
  typedef bf16x4 v4;
  typedef bf16x2 v2;
  static __device__ __forceinline__ f32x16 mfma32(v8 a, v8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ f32x4 mfma16(v8 a, v8 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float add_pair(v2 p, float acc) {
    const v2 ones = {(bf16)1.0f, (bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(p, ones, acc, false);
  }
  static __device__ __forceinline__ float dot2(v2 a, v2 b, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(a, b, acc, false);
  }
};

// Round-to-nearest-even conversion of two fp32 values to a packed pair of T.
template <typename T>
__device__ __forceinline__ typename Elem<T>::v2 cvt2(float a, float b) {
  f32x2 v = {a, b};
  return __builtin_convertvector(v, typename Elem<T>::v2);
}

// ReLU of packed fp16 / bf16 values after the conversion (rounding keeps the sign, so relu(round(x)) =
// round(relu(x))): as signed 16-bit integers the negative values are exactly those with the sign bit, so one
// packed integer max against zero per two values does it for either format (v_pk_max_i16).
template <typename V>
__device__ __forceinline__ V relu_packed(V v) {
  typedef __attribute__((ext_vector_type(sizeof(V) / 2))) short S;
  S s = __builtin_bit_cast(S, v);
  const S z = {};
  s = __builtin_elementwise_max(s, z);
  return __builtin_bit_cast(V, s);
}

// The same with the switch in a register: thr = relu_packed_threshold(on) is zero (ReLU) or the most negative
// 16-bit integer in every half (identity), so a run-time flag costs no select.
__device__ __forceinline__ unsigned relu_packed_threshold(bool on) { return on ? 0u : 0x80008000u; }
template <typename V>
__device__ __forceinline__ V relu_packed(V v, unsigned thr) {
  typedef __attribute__((ext_vector_type(sizeof(V) / 2))) short S;
  typedef __attribute__((ext_vector_type(sizeof(V) / 4))) unsigned U;
  U t;
  for (unsigned i = 0; i < sizeof(V) / 4; ++i) t[i] = thr;
  S s = __builtin_bit_cast(S, v);
  s = __builtin_elementwise_max(s, __builtin_bit_cast(S, t));
  return __builtin_bit_cast(V, s);
}

// LDS transpose read (gfx950 ds_read_b64_tr_b16).  Within each group of 16
// lanes, lane i receives for j=0..3 the 16-bit element (i%4) of the 64-bit
// word addressed by lane 4*j + i/4 of the same group.  If lane s of a group
// points at Mat[r0 + s/4][c0 + 4*(s%4)] of a row-major 16-bit matrix, lane i
// receives Mat[r0 + 0..3][c0 + i]: a 4x16 block read column-wise.
template <typename T>
__device__ __forceinline__ typename Elem<T>::v4 lds_read_tr4(const T* p) {
  s16x4 r = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DITTO_LDS s16x4*)p);
  return __builtin_bit_cast(typename Elem<T>::v4, r);
}

// x where `gone` is 0, -infinity where it is all ones (gone = (limit - 1 - index) >> 31 for "index >= limit").  A select
// by integer arithmetic: the comparisons of a masked tile are otherwise all made first and their lane masks held in
// scalar registers together, which the walks of the chain kernels do not have to spare (spills, a scratch segment).
__device__ __forceinline__ float neg_inf_where(float x, int gone) {
  return __builtin_bit_cast(float, (__builtin_bit_cast(int, x) & ~gone) | ((int)0xff800000 & gone));
}

template <typename V4, typename V8>
__device__ __forceinline__ V8 concat4(V4 lo, V4 hi) {
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Exchange across the two half-waves.  v_permlane32_swap a, b swaps a[32..63] with
// b[0..31]; started from a == b == x it leaves (a, b) = (x[l], x[l+32]) in lanes 0..31
// and (x[l-32], x[l]) in lanes 32..63, i.e. every lane holds its own value and its
// partner's.  Issued as inline asm: the compiler's builtin folds the two results into
// one value when both operands start equal.  The s_nop covers the VALU-write ->
// permlane-read hazard the compiler would otherwise pad itself.
__device__ __forceinline__ void pair_both(float x, float& a, float& b) {
  a = x;
  b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ float pair_max(float x) {
  float a, b;
  pair_both(x, a, b);
  return fmaxf(a, b);
}
__device__ __forceinline__ float pair_sum(float x) {
  float a, b;
  pair_both(x, a, b);
  return a + b;
}

// Direct global -> LDS load of 16 bytes per lane (buffer_load_dwordx4 ... lds): lane l's data
// lands at LDS byte address lds_base + 16*l; reads whose offset is at or past the resource's
// num_records return zero.  Issued as inline asm so that the compiler does not track it: its
// own bookkeeping would make every later LDS read wait for ALL outstanding loads (it cannot
// prove that the tile being filled and the tile being read are different), which serialises
// the prefetch.  The caller must s_waitcnt vmcnt(0) (and barrier) before reading the tile.
__device__ __forceinline__ void lds_dma_16(i32x4 rsrc, unsigned voffset, unsigned lds_base) {
  asm volatile(
      "s_mov_b32 m0, %2\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %0, %1, 0 offen lds"
      :
      : "v"(voffset), "s"(rsrc), "s"(lds_base)
      : "memory", "m0");
}
// The same with the LDS address given as a wave-uniform base plus a constant known once the call is inlined: a
// kernel that fills many tile slots keeps one base register instead of one address register per slot and load.
__device__ __forceinline__ void lds_dma_16_at(i32x4 rsrc, unsigned voffset, unsigned lds_base, int const_off) {
  asm volatile(
      "s_add_u32 m0, %2, %3\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %0, %1, 0 offen lds"
      :
      : "v"(voffset), "s"(rsrc), "s"(lds_base), "i"(const_off)
      : "memory", "m0", "scc");
}
// raw buffer resource (stride 0, range checked against `bytes`) as four dwords
__device__ __forceinline__ i32x4 make_rsrc(const void* base, unsigned bytes) {
  const unsigned long long a = reinterpret_cast<unsigned long long>(base);
  i32x4 r = {(int)(unsigned)a, (int)(unsigned)((a >> 32) & 0xffff), (int)bytes, 0x00020000};
  return r;
}

// Same, for a base/extent computed inside a loop: the compiler's divergence analysis can lose
// track of their uniformity, and a descriptor must live in SGPRs.
__device__ __forceinline__ i32x4 make_rsrc_uniform(const void* base, unsigned bytes) {
  const unsigned long long a = reinterpret_cast<unsigned long long>(base);
  i32x4 r = {__builtin_amdgcn_readfirstlane((int)(unsigned)a),
             __builtin_amdgcn_readfirstlane((int)(unsigned)((a >> 32) & 0xffff)),
             __builtin_amdgcn_readfirstlane((int)bytes), 0x00020000};
  return r;
}

// Cache policy for streamed output stores (buffer-store aux bits sc0 | sc1): write-through.  Left dirty in L2 a
// large output is written back in a burst after the last wave has finished; written through it streams to memory
// while the kernel still computes.  Worth 15 % on the depthwise row kernel (17.0 -> 14.4 us per call) and 11 % on
// the conv3x3 -> conv1x1 row pipeline (21.7 -> 19.2 us) once that kernel's store windows ended on whole 128-byte
// lines - with half-written lines the two halves went out separately and back-to-back launches got slower
// (22.9 -> 26.5 us); the non-temporal hint was slower on both.
constexpr int kStoreWriteThrough = 17;

// Workgroup barrier for waves that hand data to each other through LDS: waits for this wave's own LDS
// accesses first.  Spelled out because the compiler's own wait in front of __syncthreads() has been seen
// missing behind LDS writes under divergent control flow at a loop's end (the next wave then read a slot
// before the write had landed).
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// __syncthreads() behind an explicit wait for this wave's own LDS accesses, for the same reason: the generated
// code of the tile kernels had barriers that a wave with all lanes masked off in the store blocks could reach with
// its turn-around writes still in flight.
__device__ __forceinline__ void wg_sync() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __syncthreads();
}

// Output path of the BMM chain kernels.  A lane holds 4 contiguous columns of several tiles of one row and
// neighbouring lanes hold different rows: stored from registers that is 8 bytes per 128-byte line and lane, the slowest
// pattern of the store path (14 us of the 64 x 4096 x 128 attention launch; 16 bytes per line and lane move 2.9 TB/s
// over the device, 64 contiguous bytes and more per group of lanes 6 - 7 TB/s).  With a 16-bit output whose rows are
// whole 16-byte vectors a wave instead parks its ROWS x D tile in LDS, [row][2 D + 16 bytes] (the 16: the rows one
// write instruction touches spread over the banks), and this stores it row by row, 16 bytes per lane.
template <int D>
__host__ __device__ constexpr int tile_row_bytes() { return 2 * D + 16; }

// The stores are written through (see kStoreWriteThrough): they come at the very end of a workgroup's life, and lines
// left dirty in L2 would be written back by the release at the end of the dispatch, after the last wave (0.9 us of a
// 12 us launch on 96 x 512 x 64; 0.4 % of the 430 us launch on 64 x 4096 x 128).
template <typename T, int D, int ROWS>
__device__ __forceinline__ void store_tile_rows(const char* tw, T* f0, long long f_rs, int rows_valid, int N, int lane) {
  typedef typename Elem<T>::v8 V8;
  constexpr int CPR = D / 8;  // 16-byte chunks per row
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the reads are this wave's own writes of other lanes
#pragma unroll
  for (int i = 0; i < ROWS * CPR / 64; ++i) {
    const int v = 64 * i + lane, r = v / CPR, ch = v - r * CPR;
    const V8 x = *reinterpret_cast<const V8*>(tw + r * tile_row_bytes<D>() + ch * 16);
    if (r < rows_valid && 8 * ch < N) {
      V8* const dst = reinterpret_cast<V8*>(f0 + (long long)r * f_rs + 8 * ch);
      asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(dst), "v"(x) : "memory");
    }
  }
}

// Workgroups are dealt round-robin to the 8 XCDs (each with a private L2) by
// linear id.  Remap so that ids that are neighbours in the logical order (and
// share operands) land on the same XCD.
__device__ __forceinline__ unsigned xcd_remap(unsigned bid, unsigned nblk) {
  const unsigned NX = 8;
  if (nblk % NX != 0) return bid;
  return (bid % NX) * (nblk / NX) + bid / NX;
}

}  // namespace ditto
