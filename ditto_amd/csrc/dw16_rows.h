// Depthwise conv(3x3, pad 1, stride 1, SIXTEEN outputs per input channel) -> cast|relu -> conv(1x1) on NCHW
// fp16 / bf16 tensors with at most 32 input channels (512 intermediate) and 64 output channels and image
// rows of at most 120 pixels (whole 16-byte vectors): the reference's small-channel MobileNet chain,
// benchmark/chimera/cuda/depthwise3x3_conv1x1_small_channel_cuda.py:77-169 with its default `factor` = 16.
//
// At that multiplier the chain is matrix work (9 + 64 multiply-adds per intermediate value, 512 of them per
// pixel), so both stages run on the matrix cores as in dw_conv_mfma_kernel: the depthwise stage of two input
// channels is a 32x32x16 MFMA with a block-diagonal filter operand (taps 0..7, then the ninth), whose result,
// converted, IS the operand of the 1x1 stage -- the intermediate never leaves registers.  What differs is
// everything around that unit, which cost two thirds of the tiled kernel's time:
//
//  * A workgroup owns a band of output rows of one image and takes its pixels as ONE stream (an NCHW plane is
//    contiguous, so 32 consecutive pixels of the stream are 64 contiguous bytes of every output channel,
//    whatever rows they lie in).  Eight compute waves take the 32-pixel tiles of the stream round-robin, a round
//    of eight tiles between two barriers; with 14 rows of 112 pixels that is 49 tiles per workgroup and 256
//    workgroups (16 x 16 tiles: 7 rounds of workgroups for 6.1 rounds of work).
//  * Input rows arrive in a ring of LDS row slots, [channel][W + 8] per row (the 16-byte gap behind every
//    channel row is written as zeros and serves as the right border of its channel and the left border of the
//    next; rows above and below the image are out of range and arrive as zeros), brought by a loader wave that
//    does nothing else: direct global -> LDS loads, counted exactly.  There is no halo staging through
//    registers and no border arithmetic; the loader refills the slots of rows that no tile of the current round
//    reads while the round computes.
//  * The filters are staged once: W2 by direct loads (one per row), the depthwise filters regrouped into
//    operand entries straight from memory (taps 0..7 as 16-byte entries, the ninth as a dword: its MFMA's other
//    operand registers are zeros that never change).
//  * MFMA row i of a tile is pixel 16 ((i >> 2) & 1) + 4 (i >> 3) + (i & 3), so a lane ends up with 16
//    consecutive pixels of one output channel: two 16-byte stores, no turn-around through LDS.
//  * A block's work is laid out so that no two MFMAs of a wave stand back to back: conversions, tap shifts and
//    LDS reads sit between them (operands double buffered), pinned there with empty asm statements.
//
// Non-finite inputs: as in dw_conv_mfma_kernel the zero blocks of the block-diagonal operand multiply the taps
// of the block's other input channel, so an infinity there becomes NaN in this channel's intermediates.
#pragma once
#include "common.h"

namespace ditto {

struct Dw16RowsArgs {
  const void* x;   // [N][C0][H][W]
  const void* w1;  // [16 C0][1][3][3]
  const void* w2;  // [C2][16 C0]
  void* y;         // [N][C2][H][W]
  int N, C0, H, W, C2;
  int band, bands;  // output rows per workgroup, workgroups per image
  int ring;         // input row slots in LDS: >= the rows two consecutive rounds read
  int relu_mid, relu_out;
};

constexpr int kDw16Compute = 8;    // compute waves, two per SIMD
constexpr int kDw16Waves = kDw16Compute + 1;  // and the loader
constexpr int kDw16W2S = 512 + 8;  // elements per W2 row in LDS
constexpr int kDw16Round = kDw16Compute * 32;  // pixels per round

__host__ __device__ constexpr int dw16_rows_cpc(int W) { return W / 8 + 1; }  // 16-byte chunks per channel row
__host__ __device__ constexpr int dw16_rows_ni(int C0, int W) { return (C0 * dw16_rows_cpc(W) + 63) / 64; }
// rows that two consecutive rounds read: the rows that many consecutive pixels can touch, and one above and below
__host__ __device__ constexpr int dw16_rows_ring(int W) { return (2 * kDw16Round + W - 2) / W + 1 + 2; }
// LDS: 16 zero bytes, the ring, operand entries of the depthwise filters (taps 0..7: 16 bytes, the ninth: 4 bytes;
// 32 rows per block of two input channels and 32 zero rows), W2
__host__ __device__ constexpr int dw16_rows_lds_bytes(int C0, int W) {
  return 16 + dw16_rows_ring(W) * 1024 * dw16_rows_ni(C0, W) + (((C0 + 1) / 2) * 32 + 32) * (16 + 4) + 64 * kDw16W2S * 2;
}

// operand slot k of a lane's nine taps: r0s0 r0s1 r1s0 r1s1 r2s0 r2s1 r0s2 r1s2 | r2s2 (one dword pair per filter
// row covers columns x - 1 .. x + 1; the pairs first, then the third columns)
__host__ __device__ constexpr int dw16_tap_of_k(int k) {
  return k == 0 ? 0 : k == 1 ? 1 : k == 2 ? 3 : k == 3 ? 4 : k == 4 ? 6 : k == 5 ? 7 : k == 6 ? 2 : k == 7 ? 5 : k;
}

// wait until at most k rows of NI load instructions each are outstanding
template <int NI>
__device__ __forceinline__ void dw16_rows_wait(int k) {
#define DITTO_DW16_CASE(K)                                                          \
  case K:                                                                           \
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NI * K <= 63 ? NI * K : 63) : "memory"); \
    break;
  switch (k) {
    DITTO_DW16_CASE(1)
    DITTO_DW16_CASE(2)
    DITTO_DW16_CASE(3)
    DITTO_DW16_CASE(4)
    DITTO_DW16_CASE(5)
    DITTO_DW16_CASE(6)
    DITTO_DW16_CASE(7)
    DITTO_DW16_CASE(8)
    DITTO_DW16_CASE(9)
    DITTO_DW16_CASE(10)
    DITTO_DW16_CASE(11)
    DITTO_DW16_CASE(12)
    default:
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
#undef DITTO_DW16_CASE
}

template <typename T, int NI, bool RELU>
__global__ __launch_bounds__(64 * kDw16Waves) void dw16_rows_kernel(Dw16RowsArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v2 V2;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  constexpr int SLOT = 1024 * NI;
  constexpr unsigned kOut = 0x7fffffffu;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int W = p.W, H = p.H;
  const int CPC = dw16_rows_cpc(W), CS = 16 * CPC;  // chunks / bytes per channel row in LDS
  const int ring = p.ring, nblk = (p.C0 + 1) >> 1;
  const unsigned wg = xcd_remap(blockIdx.x, gridDim.x);
  const int n = (int)wg / p.bands, y0 = ((int)wg - n * p.bands) * p.band;
  const int nout = H - y0 < p.band ? H - y0 : p.band;  // output rows of this band
  const int nin = nout + 2;                            // input rows y0 - 1 .. y0 + nout
  const int npx = nout * W;                            // pixels of the band's stream
  const int ntiles = (npx + 31) >> 5, nrounds = (ntiles + kDw16Compute - 1) / kDw16Compute;
  const long long plane = (long long)H * W;
  const unsigned lds0 = (unsigned)(size_t)(DITTO_LDS char*)smem_raw;
  char* const rows = smem_raw + 16;
  uint4* const W1h = reinterpret_cast<uint4*>(rows + ring * SLOT);
  const int zero_entry = nblk * 32;
  unsigned* const A2h = reinterpret_cast<unsigned*>(W1h + zero_entry + 32);
  T* const W2s = reinterpret_cast<T*>(A2h + zero_entry + 32);
  const float inv_w = 1.0f / (float)W, inv_ring = 1.0f / (float)ring;
  // last input row (band relative: row k is image row y0 - 1 + k) that round rd reads
  auto last_row = [&](int rd) __attribute__((always_inline)) {
    int e = kDw16Round * rd + kDw16Round - 1;
    if (e > npx - 1) e = npx - 1;
    return (int)(((float)e + 0.5f) * inv_w) + 2;  // exact: the host keeps H * W below 2^20
  };

  if (wave == kDw16Compute) {
    // ======================= loader wave =======================
    // instruction i of a row: lane l brings 16 bytes of job 64 i + l = channel * CPC + chunk
    const i32x4 rsrc = make_rsrc_uniform(reinterpret_cast<const T*>(p.x) + (long long)n * p.C0 * plane,
                                         (unsigned)(p.C0 * plane * 2));
    const float inv_cpc = 1.0f / (float)CPC;
    unsigned vo[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int job = 64 * i + lane;
      const int c = (int)(((float)job + 0.5f) * inv_cpc), chunk = job - c * CPC;
      vo[i] = (c < p.C0 && chunk < CPC - 1) ? (unsigned)(c * (int)plane * 2 + chunk * 16) : kOut;
    }
    int slot = 0;  // of the next row to issue: rows are issued in order, row k goes to slot k % ring
    auto issue = [&](int k) __attribute__((always_inline)) {
      const int y = y0 - 1 + k;
      const bool ok = y >= 0 && y < H;
      const unsigned shift = (unsigned)(y * W * 2);
      const unsigned dst = lds0 + 16 + (unsigned)(slot * SLOT);
#pragma unroll
      for (int i = 0; i < NI; ++i) lds_dma_16(rsrc, ok ? vo[i] + shift : kOut, dst + 1024 * i);
      slot = slot + 1 == ring ? 0 : slot + 1;
    };
    constexpr int AH = 63 / NI < 12 ? 63 / NI : 12;  // rows in flight at most
    int issued = 0;
    while (issued < nin && issued < ring && issued < AH) issue(issued++);
    for (int rd = 0; rd < nrounds; ++rd) {
      // rows up to `need` are read in round rd: rows still in flight after them may stay in flight
      int need = last_row(rd);
      if (need > nin - 1) need = nin - 1;
      while (issued <= need) {  // (the counter let fewer rows start than the round reads)
        dw16_rows_wait<NI>(AH - 1);
        issue(issued++);
      }
      int k = issued - 1 - need;
      dw16_rows_wait<NI>(k);
      lds_barrier();
      // Every compute wave has finished round rd - 1.  Row k2 goes where row k2 - ring was: that one must lie
      // above the first row round rd reads.
      const int first = (int)(((float)(kDw16Round * rd) + 0.5f) * inv_w);
      while (issued < nin && issued - ring < first && k < AH) {
        issue(issued++);
        ++k;
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }

  // ======================= compute waves =======================
  const int ln = lane & 31, g = lane >> 5;
  // ---- the filters, once
  if (tid < 4) reinterpret_cast<unsigned*>(smem_raw)[tid] = 0u;  // left border of channel 0 in ring slot 0
  {
    // W2 rows by direct loads: row c2 is 1 KB at most (512 intermediate channels), one instruction
    const i32x4 w2_rsrc = make_rsrc_uniform(p.w2, (unsigned)(p.C2 * p.C0 * 16 * 2));
    const unsigned row_bytes = (unsigned)(p.C0 * 16 * 2);
    const unsigned w2_lds = (unsigned)(size_t)(DITTO_LDS char*)W2s;
    for (int c2 = wave; c2 < 64; c2 += kDw16Compute) {
      const unsigned vo = (c2 < p.C2 && 16u * lane < row_bytes) ? c2 * row_bytes + 16u * lane : kOut;
      lds_dma_16(w2_rsrc, vo, w2_lds + (unsigned)(c2 * kDw16W2S * 2));
    }
    // depthwise filters as A-operand entries: row m = 16 h + 8 a + 4 gg + b of a block is its intermediate
    // channel 16 h + 8 gg + 4 a + b, so that accumulator registers 8 s .. 8 s + 7 of a lane are 8 consecutive
    // channels; entry (blk, m): taps 0 .. 7 in gather order, and the ninth tap in a table of its own
    const unsigned short* W1g = reinterpret_cast<const unsigned short*>(p.w1);
    const int C1 = 16 * p.C0;
    for (int e = tid; e < nblk * 32; e += 64 * kDw16Compute) {
      const int m = e & 31, blk = e >> 5;
      const int mm = m & 15;
      const int cml = 32 * blk + 16 * (m >> 4) + 8 * ((mm >> 2) & 1) + 4 * (mm >> 3) + (mm & 3);
      unsigned raw[9];
#pragma unroll
      for (int i = 0; i < 9; ++i) raw[i] = cml < C1 ? W1g[cml * 9 + dw16_tap_of_k(i)] : 0u;
      W1h[e] = uint4{raw[0] | (raw[1] << 16), raw[2] | (raw[3] << 16), raw[4] | (raw[5] << 16), raw[6] | (raw[7] << 16)};
      A2h[e] = raw[8];
    }
    if (tid < 32) {
      W1h[zero_entry + tid] = uint4{0, 0, 0, 0};
      A2h[zero_entry + tid] = 0;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  // A-operand entries of this lane: its own half of the block diagonal, zeros else
  // (byte offsets from the start of LDS: 32-bit address arithmetic)
  const bool own_half = (ln >> 4) == g;
  const int w1h_off = 16 + ring * SLOT, a2h_off = w1h_off + (zero_entry + 32) * 16, w2s_off = a2h_off + (zero_entry + 32) * 4;
  const int a1_base = w1h_off + (own_half ? 16 * ln : 16 * zero_entry);
  const int a2_base = a2h_off + (own_half ? 4 * ln : 4 * zero_entry);
  const int own_mask = own_half ? -1 : 0;  // block blk's entries: + 512 blk (+ 128 blk) bytes for the lanes that have any
  // pixel of this lane inside a tile (as a column of the depthwise MFMA and a row of the 1x1 MFMA)
  const int pix = 16 * ((ln >> 2) & 1) + 4 * (ln >> 3) + (ln & 3);
  const int cs2 = 2 * CS;
  const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      reinterpret_cast<T*>(p.y) + (long long)n * p.C2 * plane, 0, (int)(p.C2 * plane * 2), 0x00020000);
  const int last = nblk - 1;
  const int w2_ln = w2s_off + ln * kDw16W2S * 2 + 16 * g;  // this lane's row and k group inside a 32-row tile of W2

  for (int rd = 0; rd < nrounds; ++rd) {
    lds_barrier();  // the rows this round reads have landed (round 0: the filters are staged)
    const int tile = kDw16Compute * rd + wave;
    if (tile >= ntiles) continue;  // wave-uniform
    // ---- the lane's pixel: row yy of the band, column x; its taps' dword pairs in the three ring rows
    int pl = 32 * tile + pix;
    if (pl > npx - 1) pl = npx - 1;  // past the band's end: computed and not stored
    const int yy = (int)(((float)pl + 0.5f) * inv_w), x = pl - yy * W;
    const unsigned sh = (unsigned)((x - 1) & 1) * 16u;
    int xa[3];
    int sl = yy - ring * (int)(((float)yy + 0.5f) * inv_ring);  // yy % ring
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      xa[r] = 16 + sl * SLOT + g * CS + ((x - 1) & ~1) * 2;
      sl = sl + 1 == ring ? 0 : sl + 1;
    }

    f32x16 o[2], acc;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[t][r] = 0.f;
    V8 a1n, b1n, wf[2][2][2], pf[2][2];
    // operands of the ninth tap's MFMA: only the first of their four registers ever changes
    u32x4 a2u = {0u, 0u, 0u, 0u}, b2u = {0u, 0u, 0u, 0u};
    unsigned d0[3], d1[3];
    auto load_w2 = [&](int blk, int buf) __attribute__((always_inline)) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int s = 0; s < 2; ++s)
          wf[buf][t][s] = *reinterpret_cast<const V8*>(smem_raw + (w2_ln + 64 * blk) + (32 * t * kDw16W2S * 2 + 32 * s));
    };
    auto load_a = [&](int blk) __attribute__((always_inline)) {
      a1n = *reinterpret_cast<const V8*>(smem_raw + (a1_base + ((blk << 9) & own_mask)));
      a2u[0] = *reinterpret_cast<const unsigned*>(smem_raw + (a2_base + ((blk << 7) & own_mask)));
      asm volatile("" : "+v"(a2u));  // in place: the other three registers stay the zeros they are
    };
    // the taps of block blk: the dword pairs are read early (read_b) and shifted into operand order late (make_b)
    auto read_b = [&](int blk) __attribute__((always_inline)) {
#pragma unroll
      for (int r = 0; r < 3; ++r) {
        const unsigned* xw = reinterpret_cast<const unsigned*>(smem_raw + (xa[r] + blk * cs2));
        d0[r] = xw[0];
        d1[r] = xw[1];
      }
    };
    auto make_b = [&]() __attribute__((always_inline)) {
      unsigned p01[3], t2[3];
#pragma unroll
      for (int r = 0; r < 3; ++r) {
        p01[r] = __builtin_amdgcn_alignbit(d1[r], d0[r], sh);  // columns x - 1, x
        t2[r] = __builtin_amdgcn_alignbit(0u, d1[r], sh);      // column x + 1 in the low half
      }
      const u32x4 b1r = {p01[0], p01[1], p01[2], __builtin_amdgcn_perm(t2[1], t2[0], 0x05040100u)};
      b1n = __builtin_bit_cast(V8, b1r);
      b2u[0] = t2[2] & 0xffffu;
      // (plain arithmetic is free to sink to its use: the empty asm keeps it here, between two MFMAs)
      asm volatile("" : "+v"(b1n), "+v"(b2u));
    };
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    auto depthwise_a = [&]() __attribute__((always_inline)) { acc = Elem<T>::mfma32(a1n, b1n, zero16); };
    auto depthwise_b = [&]() __attribute__((always_inline)) {
      acc = Elem<T>::mfma32(__builtin_bit_cast(V8, a2u), __builtin_bit_cast(V8, b2u), acc);
    };
    auto convert = [&](int s, int buf) __attribute__((always_inline)) {  // half s of the block in `acc`
      const V2 c0v = cvt2<T>(acc[8 * s + 0], acc[8 * s + 1]), c1v = cvt2<T>(acc[8 * s + 2], acc[8 * s + 3]);
      const V2 c2v = cvt2<T>(acc[8 * s + 4], acc[8 * s + 5]), c3v = cvt2<T>(acc[8 * s + 6], acc[8 * s + 7]);
      pf[buf][s] = V8{c0v[0], c0v[1], c1v[0], c1v[1], c2v[0], c2v[1], c3v[0], c3v[1]};
      if (RELU) pf[buf][s] = relu_packed(pf[buf][s]);
      asm volatile("" : "+v"(pf[buf][s]));
    };
    // rows = pixels, columns = output channels
    auto pointwise = [&](int t, int s, int buf) __attribute__((always_inline)) {
      o[t] = Elem<T>::mfma32(pf[buf][s], wf[buf][t][s], o[t]);
    };
#define DITTO_SB __builtin_amdgcn_sched_barrier(0)
    // Software pipeline over blocks of 32 intermediate channels (two input channels): while the 1x1 MFMAs of block b
    // issue, the depthwise result of b + 1 is converted (into the other operand buffer), the taps of b + 2 are
    // shifted into place and the depthwise MFMAs of b + 2 follow; the taps of b + 3 are read between those two.
    // Blocks past the end recompute the last one.
    auto clampb = [&](int b) __attribute__((always_inline)) { return b < last ? b : last; };
    load_a(0);
    load_w2(0, 0);
    read_b(0);
    make_b();
    read_b(clampb(1));
    depthwise_a();
    depthwise_b();
    load_a(clampb(1));
    convert(0, 0);
    convert(1, 0);
    make_b();
    read_b(clampb(2));
    depthwise_a();
    depthwise_b();
    DITTO_SB;
    for (int blk = 0; blk < nblk; blk += 2) {
#pragma unroll
      for (int u = 0; u < 2; ++u) {  // (unrolled by two: the operand buffers alternate)
        const int b = blk + u;
        if (b >= nblk) break;
        const int cur = u, oth = u ^ 1;
        load_a(clampb(b + 2));
        load_w2(clampb(b + 1), oth);
        DITTO_SB;
        pointwise(0, 0, cur); DITTO_SB; convert(0, oth); DITTO_SB;
        pointwise(1, 0, cur); DITTO_SB; convert(1, oth); DITTO_SB;
        pointwise(0, 1, cur); DITTO_SB; make_b(); DITTO_SB;
        pointwise(1, 1, cur); DITTO_SB;
        depthwise_a(); DITTO_SB;
        read_b(clampb(b + 3)); DITTO_SB;
        depthwise_b(); DITTO_SB;
      }
    }
#undef DITTO_SB
    // ---- output: o[t][i] = out[pixel 16 g + i of the tile][c2 = 32 t + ln]
    const int px0 = 32 * tile + 16 * g;
    const unsigned soff = (unsigned)((y0 * W + 32 * tile) * 2);  // wave-uniform part of the address
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int c2 = 32 * t + ln;
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = o[t][8 * hh + e];
        const V2 q0 = cvt2<T>(v[0], v[1]), q1 = cvt2<T>(v[2], v[3]), q2 = cvt2<T>(v[4], v[5]), q3 = cvt2<T>(v[6], v[7]);
        V8 px8 = {q0[0], q0[1], q1[0], q1[1], q2[0], q2[1], q3[0], q3[1]};
        if (p.relu_out) px8 = relu_packed(px8);
        const unsigned vo = (c2 < p.C2 && px0 + 8 * hh < npx) ? (unsigned)(c2 * (int)plane * 2 + 32 * g + 16 * hh) : kOut;
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, px8), y_rsrc, vo, soff, 0);
      }
    }
  }
#else
  (void)p;
#endif
}

template <typename T, int NI, bool RELU>
hipError_t launch_dw16_rows_ni(const Dw16RowsArgs& args, hipStream_t stream) {
  const int lds = dw16_rows_lds_bytes(args.C0, args.W);
  auto kern = dw16_rows_kernel<T, NI, RELU>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(args.N * args.bands)), dim3(64 * kDw16Waves), lds, stream, args);
  return hipGetLastError();
}

template <typename T>
hipError_t launch_dw16_rows(const Dw16RowsArgs& args, hipStream_t stream) {
  switch (dw16_rows_ni(args.C0, args.W)) {
    case 1: return args.relu_mid ? launch_dw16_rows_ni<T, 1, true>(args, stream) : launch_dw16_rows_ni<T, 1, false>(args, stream);
    case 2: return args.relu_mid ? launch_dw16_rows_ni<T, 2, true>(args, stream) : launch_dw16_rows_ni<T, 2, false>(args, stream);
    case 3: return args.relu_mid ? launch_dw16_rows_ni<T, 3, true>(args, stream) : launch_dw16_rows_ni<T, 3, false>(args, stream);
    case 4: return args.relu_mid ? launch_dw16_rows_ni<T, 4, true>(args, stream) : launch_dw16_rows_ni<T, 4, false>(args, stream);
    case 5: return args.relu_mid ? launch_dw16_rows_ni<T, 5, true>(args, stream) : launch_dw16_rows_ni<T, 5, false>(args, stream);
    case 6: return args.relu_mid ? launch_dw16_rows_ni<T, 6, true>(args, stream) : launch_dw16_rows_ni<T, 6, false>(args, stream);
    case 7: return args.relu_mid ? launch_dw16_rows_ni<T, 7, true>(args, stream) : launch_dw16_rows_ni<T, 7, false>(args, stream);
    case 8: return args.relu_mid ? launch_dw16_rows_ni<T, 8, true>(args, stream) : launch_dw16_rows_ni<T, 8, false>(args, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace ditto
