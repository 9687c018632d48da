// conv(3x3, pad 1, stride 1) -> cast|relu -> conv(1x1) on NCHW fp16 / bf16 tensors with at most 64 input
// and intermediate channels, at most 256 output channels and image rows of at most 64 pixels (whole
// 16-byte vectors), 16-bit output: the bottleneck block of a ResNet-50 at 56 x 56.  With the template flag F13
// the same pipeline runs conv(1x1) -> cast|relu -> conv(3x3, pad 1) with at most 64 channels everywhere (described
// at the kernel).
//
// Reference chain: benchmark/chimera/cuda/conv_relu_conv_relu... / testing/hyper_fusion/
// conv_relu_conv_relu_fuse_hw_cuda.py (conv3x3 -> conv1x1, the second GEMM consuming the first one's tile).
//
// The chain is bound by its output traffic (256 channels out for 64 in), so the kernel is built as a
// pipeline over image rows whose stages run on waves of their own inside one workgroup, and the output
// stores start as soon as the first rows are through instead of after the whole tile:
//
//  * A workgroup owns a band of output rows of one image.  ALL input rows of the band (band + 2) are
//    issued at kernel start as direct global -> LDS loads ([channel][W] per row; rows outside the image
//    are out of range and arrive as zeros): rows 0..3 by waves 0..3 ahead of their W1 fragments, rows
//    4 and 5 by waves 4 and 5, the rest by waves 6 and 7 - waves 4..7 have nothing to store before step 1
//    and wait for their rows before then, so every counter wait is exact.  Waves 0..3 turn the rows round
//    into Xt[pixel + 1][64 channels] (a ring of 6 rows with a zero pixel left and right, 16-byte chunks
//    XOR-swizzled by pixel pair so that 16 consecutive pixels cover every LDS bank once) with the
//    transposing LDS read, one step before the row is needed.
//  * Step k = output rows 2k, 2k + 1.  First convolution on waves 0..3 = (row, half of the intermediate
//    channels): mid^T[c1][pixel] = W1 . X as 36 x 2 MFMAs 32x32x16 with the wave's 36 W1 fragments
//    RESIDENT IN REGISTERS (loaded once from the repacked copy in the workspace) and the pixel
//    fragments read from Xt at the tap's offset; the cast result goes to LDS as mid[pixel][64]
//    (three buffers).
//  * Second convolution of the previous step on waves 4..7 (64 output channels each, W2 fragments in
//    registers, one wave per SIMD next to a first-convolution wave): out^T[c2][pixel] = W2 . mid as
//    16x16x32 MFMAs whose column j of tile t is pixel 8 j + t of a window of the band's pixels, so a lane
//    ends with 8 consecutive pixels of each of its 4 channels and the 16 lanes of a column group store
//    256 contiguous bytes of a channel plane with one 16-byte store each; the windows end on whole
//    128-byte lines.
//  One barrier per step; the only waves that wait for memory after the prologue are waves 4..7, in the
//  store queue.
#pragma once
#include "common.h"

namespace ditto {

struct ConvRowsArgs {
  const void* x;    // [N][C0][H][W]
  const void* w1f;  // W1 as MFMA fragments [tap][c0 / 16][c1 / 32][lane][8] (pack_conv_w2_resident's layout)
  const void* w2;   // [C2][C1]
  void* y;          // [N][C2][H][W]
  int N, C0, H, W, C1, C2;
  int band, bands;  // output rows per workgroup, workgroups per image
  int relu_mid, relu_out;
  // conv(1x1) -> cast|relu -> conv(3x3, pad 1) through the same pipeline (see F13 below): w1x the 1x1 weights
  // [Cm][C0], relu_pre the ReLU between the two; w1f then holds the 3x3 weights [C1][Cm][3][3] as fragments,
  // C1 = C2 the output channels (at most 64), relu_mid the ReLU of the output
  const void* w1x;
  int f13, Cm, relu_pre;
};

constexpr int kCvrC = 64;      // input / intermediate channels (padded)
constexpr int kCvrWaves = 8;   // four load / first-convolution waves, four second-convolution / store waves
constexpr int kCvrRing = 6;    // rows of the transposed ring
constexpr int kCvrW1Bytes = 9 * kCvrC * kCvrC * 2;

// LDS: band + 2 raw rows of 128 W bytes, the ring of transposed rows, three intermediate steps of 2 W pixels
// (and, for the 1x1 -> 3x3 chain, the 1x1 weights as 8 fragments of 1 KB)
constexpr int kCvrW1xBytes = 2 * 4 * 1024;
__host__ __device__ constexpr int conv_rows_lds_bytes(int W, int band, bool f13 = false) {
  return (band + 2) * 128 * W + kCvrRing * (W + 2) * 128 + 3 * (2 * W) * 128 + (f13 ? kCvrW1xBytes : 0);
}
// waves 6 and 7 keep half each of the band's rows from the seventh on in flight at once, W / 8 load instructions
// per row, next to the 8 loads of their W2 fragments: stay inside the 6-bit outstanding-load counter
__host__ __device__ constexpr int conv_rows_band_max(int W) { return 2 * (48 / (W / 8)) + 4; }

// F13: the chain conv(1x1) -> cast|relu -> conv(3x3, pad 1) with at most 64 channels everywhere (the reference's
// benchmark/chimera/cuda/conv1x1_conv3x3_cuda.py row).  The 3x3 convolution takes the place of the pipeline's first
// convolution, so its input - the 1x1 convolution's result - is what the ring of transposed rows has to hold:
// instead of only turning a raw row round, the transposing stage multiplies the transposed fragments by the 1x1
// weights (fragments in LDS, 8 MFMAs 32x32x16 per 32 pixels) and writes the cast result into the ring; rows outside
// the image arrive as zeros and stay zeros, which is the 3x3 convolution's padding.  The pipeline's second stage
// has no convolution left: waves 4..7 take 16 output channels each and multiply by an identity fragment, which
// leaves the values as they are (one 16-bit rounding, done where the 3x3 result is cast) and gives the
// 8-consecutive-pixel store layout.  (A non-finite output value turns the other channels of its pixel that share
// the fragment into NaN: 0 x inf.)  With so little left to do there, waves 4..7 also run the transposing stage -
// two waves per row, one per pixel tile of 32, next to the MFMA loop of waves 0..3 (for rows 0..3, which are needed
// first, all eight waves share it) - at a raised wave priority.
template <typename T, int NI, bool F13>
__global__ __launch_bounds__(64 * kCvrWaves) void conv_rows_kernel(ConvRowsArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  typedef typename Elem<T>::v2 V2;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  constexpr unsigned kOut = 0x7fffffffu;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int Wi = p.W, H = p.H;
  const int MW = Wi + 2, SJ = Wi >> 2;  // pixels of a transposed row; strips of 8 pixels in a step of two rows
  const int RAWROW = 128 * Wi, XTROW = MW * 128, MIDBUF = 2 * Wi * 128;
  const unsigned wg = xcd_remap(blockIdx.x, gridDim.x);
  const int n = (int)wg / p.bands, y0 = ((int)wg - n * p.bands) * p.band;
  const int nout = H - y0 < p.band ? H - y0 : p.band;
  const int nin = nout + 2;
  const int nsteps = (nout + 1) >> 1;
  const long long plane = (long long)H * Wi;
  char* const raw = smem_raw;
  char* const Xt = raw + (p.band + 2) * RAWROW;
  char* const mid = Xt + kCvrRing * XTROW;
  char* const w1x = mid + 3 * MIDBUF;  // F13: fragment (ct, kk) of the 1x1 weights at ((4 ct + kk) * 64 + lane) * 16
  const unsigned lds0 = (unsigned)(size_t)(DITTO_LDS char*)smem_raw;

  // direct global -> LDS load of input row q of the band (band-relative; image row y0 - 1 + q)
  const i32x4 x_rsrc = make_rsrc_uniform(reinterpret_cast<const T*>(p.x) + (long long)n * p.C0 * plane,
                                         (unsigned)(p.C0 * plane * 2));
  auto issue_row = [&](int q) __attribute__((always_inline)) {
    const int S8 = Wi >> 3;  // 16-byte pieces per channel row
    const int y = y0 - 1 + q;
    const bool ok = y >= 0 && y < H;
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int job = 64 * i + lane, c = job / S8, piece = job - c * S8;  // channels >= C0 are out of range
      const unsigned vo = ok ? (unsigned)(c * (int)plane * 2 + piece * 16 + y * Wi * 2) : kOut;
      lds_dma_16(x_rsrc, vo, lds0 + q * RAWROW + 1024 * i);
    }
  };

  // raw row q -> ring slot q % 6: unit (pixel tile t of 32, 16 channels kk): the lane receives channels
  // 16 kk + 8 g .. + 7 of pixel 32 t + ln (two transposing reads) and writes them as one 16-byte chunk
  const int i16 = lane & 15, h = (lane >> 4) & 1;
  const int ntile = (Wi + 31) >> 5;
  // (F13: pixel tiles t0, t0 + tstep, .. only, so that two waves can share a row)
  auto transpose_row = [&](int q, int t0, int tstep) __attribute__((always_inline)) {
    const char* const src = raw + q * RAWROW;
    char* const dst = Xt + (q % kCvrRing) * XTROW;
    // per pixel tile: its reads first (one LDS round trip), then the writes
#pragma unroll 1
    for (int t = t0; t < ntile; t += tstep) {
      V8 v[4];
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const char* rd = src + (16 * kk + 8 * g + (i16 >> 2)) * (2 * Wi) + (32 * t + 16 * h + 4 * (i16 & 3)) * 2;
        const V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(rd));
        const V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(rd + 4 * 2 * Wi));
        v[kk] = concat4<V4, V8>(lo, hi);
      }
      const int px = 32 * t + ln, col = px + 1;
      if (F13) {
        // the 1x1 convolution of the 32 pixels: a[ct][4 i + e] = mid channel 32 ct + 8 i + 4 g + e of pixel px,
        // 8 bytes into chunk 4 ct + i of the pixel
        f32x16 a2[2];
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
          for (int e = 0; e < 16; ++e) a2[ct][e] = 0.f;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
#pragma unroll
          for (int ct = 0; ct < 2; ++ct)
            a2[ct] = Elem<T>::mfma32(*reinterpret_cast<const V8*>(w1x + ((4 * ct + kk) * 64 + lane) * 16), v[kk], a2[ct]);
#pragma unroll
        for (int ct = 0; ct < 2; ++ct) {
          const f32x16 a = a2[ct];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const V2 a0 = cvt2<T>(a[4 * i], a[4 * i + 1]), a1 = cvt2<T>(a[4 * i + 2], a[4 * i + 3]);
            V4 w = {a0[0], a0[1], a1[0], a1[1]};
            if (p.relu_pre) w = relu_packed(w);
            if (px < Wi) *reinterpret_cast<V4*>(dst + col * 128 + (((4 * ct + i) ^ ((col >> 1) & 7)) << 4) + 8 * g) = w;
          }
        }
      } else {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
          if (px < Wi) *reinterpret_cast<V8*>(dst + col * 128 + (((2 * kk + g) ^ ((col >> 1) & 7)) << 4)) = v[kk];
      }
    }
  };

  if (wave >= 4) {
    // ======================= second convolution / stores =======================
    // F13: these waves' short instruction streams (the 1x1 stage of a pixel tile, a window of stores) share a SIMD
    // with an MFMA loop that leaves them about one issue slot in ten cycles; with a raised priority they get
    // through in two thirds of the time (5 % of the kernel).  With the 3x3 first the same setting delays the first
    // convolution's start-up and costs 10 %.
    if (F13) __builtin_amdgcn_s_setprio(2);
    const int hh = wave - 4;  // output channels 64 hh .. 64 hh + 63 (F13: 16 hh .. 16 hh + 15)
    // (F13: the identity's rows 16 hh .. + 15 are zero outside the 32-channel block hh / 2: one k step)
    constexpr int NCT = F13 ? 1 : 4, NKS = F13 ? 1 : 2;
    const int cb = F13 ? 16 * hh : 64 * hh, ks0 = F13 ? hh >> 1 : 0;
    // Before their first store (step 1) these waves bring the input rows from the fifth on (rows 0 .. 3 are the
    // other waves'): rows 4 and 5, turned round during step 0, by waves 4 and 5, which wait for them before the
    // first barrier; the rest, turned round from step 1 on, by waves 6 and 7, which wait before the second.
    // F13: waves 6 and 7, whose rows are needed last, first fetch the 1x1 weights, four of the eight fragments
    // each - lane (ln, g) holds W1x[32 ct + ln][16 kk + 8 g .. + 7] of fragment (ct, kk) - and put them into LDS
    if (F13 && hh >= 2) {
      const T* W1g = reinterpret_cast<const T*>(p.w1x);
      V8 wx[4];
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const int c1 = 32 * (hh - 2) + ln, c0 = 16 * kk + 8 * g;
        V8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (c1 < p.Cm && c0 < p.C0) v = *reinterpret_cast<const V8*>(W1g + (long long)c1 * p.C0 + c0);
        wx[kk] = v;
      }
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) *reinterpret_cast<V8*>(w1x + ((4 * (hh - 2) + kk) * 64 + lane) * 16) = wx[kk];
    }
    if (hh < 2) {
      if (4 + hh < nin) issue_row(4 + hh);
    } else {
#pragma unroll 1
      for (int q = 4 + hh; q < nin; q += 2) issue_row(q);
    }
    const int j = lane & 15, kg = lane >> 4;
    // A operand: lane (m, kg) holds W2[64 hh + 16 ct + m][32 ks + 8 kg .. + 7]
    V8 w2f[NCT][NKS];
    {
      const T* W2g = reinterpret_cast<const T*>(p.w2);
#pragma unroll
      for (int ct = 0; ct < NCT; ++ct)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const int c2 = cb + 16 * ct + j, k0 = 32 * (ks0 + ks) + 8 * kg;
          V8 v = {0, 0, 0, 0, 0, 0, 0, 0};
          if (F13) {  // row c2 of the identity
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = k0 + e == c2 ? (T)1.0f : (T)0.0f;
          } else if (c2 < p.C2 && k0 < p.C1) {
            v = *reinterpret_cast<const V8*>(W2g + (long long)c2 * p.C1 + k0);
          }
          w2f[ct][ks] = v;
        }
    }
    if (F13) {
      lds_barrier();  // the 1x1 weights are in LDS, and rows 0 .. 3 (the other waves have waited for them)
      // the second pixel tile of rows 0 .. 3, next to the other waves' first
      if (ntile == 2 && hh < nin) transpose_row(hh, 1, 2);
    }
    // The band's output pixels, row after row, are one contiguous run of every channel plane.  After step s the
    // wave stores the pixels up to the last whole 128-byte line of what is computed (the rest waits for the next
    // step; with rows of 112 bytes every other line would else be written in two halves, 3 us apart, and go out to
    // memory twice), in windows of 128 pixels: MFMA column j of tile t is pixel w0 + 8 j + t of the band, so a
    // lane ends with 8 consecutive pixels of each of its 4 channels and 16 lanes write 256 contiguous bytes.
    // The pixel lives in the intermediate buffer of its own step (slot SJ t + jj, chunk XORed with (jj >> 1) & 7 and t),
    // this step's or the one before: three buffers.
    const int WB = 2 * Wi;                       // pixels of a step
    const int align = WB >= 64 ? 64 : 8;         // window ends on whole lines where a step spans one
    const int A0 = y0 * Wi;                      // the band's first pixel inside a channel plane
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<T*>(p.y) + (long long)n * p.C2 * plane, 0, (int)(p.C2 * plane * 2), 0x00020000);
    int ws = 0;  // first pixel of the band not stored yet
    for (int k = 0; k <= nsteps; ++k) {
      if (k == (hh < 2 ? 0 : 1)) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's rows (and W2 fragments)
      lds_barrier();  // the intermediate rows of step k - 1 are written
      if (F13) {
        // rows 2k + 4, 2k + 5 for the next step (their ring slots were last read in step k - 1; they landed before
        // barrier k): here, next to the other waves' MFMA loop, two waves per row where it has two pixel tiles
        const int q = 2 * k + 4 + (hh & 1);
        const bool share = ntile == 2;
        if (q < nin && (share || hh < 2)) transpose_row(q, share ? hh >> 1 : 0, share ? 2 : 1);
      }
      if (k == 0 || cb >= p.C2) continue;
      const int s = k - 1;
      const int ce = (2 * (s + 1) < nout ? 2 * (s + 1) : nout) * Wi;  // pixels computed so far
      const int we = k == nsteps ? ce : ((A0 + ce) / align) * align - A0;
      for (int w0 = ws; w0 < we; w0 += 128) {
        const int q = w0 + 8 * j;                  // the lane's 8 pixels q .. q + 7
        const bool on = q < we;
        const int qc = on ? q : w0;
        const int sq = qc >= s * WB ? s : s - 1;   // the step that computed them
        const int jj = (qc - sq * WB) >> 3;
        const char* const mr = mid + (sq % 3) * MIDBUF + jj * 128;
        const int b_x = (jj >> 1) & 7;
        V8 bf[NKS][8];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
          for (int t = 0; t < 8; ++t)
            bf[ks][t] = *reinterpret_cast<const V8*>(mr + SJ * t * 128 + (((4 * (ks0 + ks) + kg) ^ b_x ^ (F13 ? t : 0)) << 4));
        const unsigned y_lane = (unsigned)((cb + 4 * kg) * (int)plane * 2 + (A0 + qc) * 2);
#pragma unroll
        for (int ct = 0; ct < NCT; ++ct) {
          if (cb + 16 * ct >= p.C2) break;  // wave-uniform
          f32x4 o[8];
          const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int t = 0; t < 8; ++t) o[t] = Elem<T>::mfma16(w2f[ct][0], bf[0][t], z);
          if (NKS == 2) {
#pragma unroll
            for (int t = 0; t < 8; ++t) o[t] = Elem<T>::mfma16(w2f[ct][NKS - 1], bf[NKS - 1][t], o[t]);
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const V2 q0 = cvt2<T>(o[0][i], o[1][i]), q1 = cvt2<T>(o[2][i], o[3][i]);
            const V2 q2 = cvt2<T>(o[4][i], o[5][i]), q3 = cvt2<T>(o[6][i], o[7][i]);
            V8 px8 = {q0[0], q0[1], q1[0], q1[1], q2[0], q2[1], q3[0], q3[1]};
            if (p.relu_out) px8 = relu_packed(px8);
            const int c2 = cb + 16 * ct + 4 * kg + i;
            const unsigned vo = (on && c2 < p.C2) ? y_lane : kOut;
            const unsigned soff = (unsigned)((16 * ct + i) * (int)plane * 2);
            __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, px8), y_rsrc, vo, soff, kStoreWriteThrough);
          }
        }
      }
      if (we > ws) ws = we;
    }
    return;
  }

  // ======================= loads, transposition and first convolution =======================
  const int rho = wave & 1, c1t = wave >> 1;
  // ---- this wave's input row of the first step: q = wave (the later rows come through waves 4 .. 7); the wave
  // issues no other memory instruction after its prologue
  if (wave < nin) issue_row(wave);
  // the zero pixels left and right of every ring row
  if (wave == 0)
    for (int i = lane; i < kCvrRing * 2 * 8; i += 64) {
      const int row = i >> 4, side = (i >> 3) & 1, piece = i & 7;
      *reinterpret_cast<i32x4*>(Xt + row * XTROW + (side ? (Wi + 1) * 128 : 0) + piece * 16) = i32x4{0, 0, 0, 0};
    }
  // the wave's fragments of W1: step st = (tap, kk), lane (ln, g) holds W1[32 c1t + ln][16 kk + 8 g .. + 7][tap]
  constexpr int NSTEP = 36;
  V8 w1f[NSTEP];
  {
    const char* w = reinterpret_cast<const char*>(p.w1f) + c1t * 1024 + lane * 16;
#pragma unroll
    for (int st = 0; st < NSTEP; ++st) w1f[st] = *reinterpret_cast<const V8*>(w + st * 2048);
  }
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NSTEP) : "memory");  // the row (issued ahead of the W1 fragments) has landed
  if (F13) lds_barrier();  // waves 6 and 7 have put the 1x1 weights into LDS
  // rows 0 .. 3: what step 0 reads (F13: a second pixel tile is the other waves')
  if (wave < nin) transpose_row(wave, 0, F13 ? 2 : 1);

  // pixel tiles pt = 0, 1: column ln of the MFMA is pixel 32 pt + ln of the row.
  // Ring rows are whole multiples of 128 bytes, so a fragment's address is (row + xb) ^ (chunk << 4) with
  // xb = column * 128 | swizzle << 4; likewise the intermediate pixel's chunk is at (buffer + mb) ^ (chunk << 4).
  // Column + 32 has the same swizzle, so the second tile's fragment lies 4096 bytes behind the first one's (an
  // immediate offset); its pixels past the row read whatever follows the ring row - the next one or the
  // intermediate buffers, inside the allocation - and their MFMA columns are dropped.
  int xb[3], mb[2];
  bool px_ok[2];
#pragma unroll
  for (int ds = 0; ds < 3; ++ds) {
    const int col = (ln < Wi ? ln : 0) + ds;
    xb[ds] = col * 128 | (((col >> 1) & 7) << 4);
  }
#pragma unroll
  for (int pt = 0; pt < 2; ++pt) {
    const int px = 32 * pt + ln;
    px_ok[pt] = px < Wi;
    const int pxc = px_ok[pt] ? px : 0;
    // pixel of the step: slot SJ t + j with 8 j + t = W rho + px
    const int pp = Wi * rho + pxc, jj = pp >> 3, tt = pp & 7;
    // (the chunk index is XORed with tt as well: the 8 lanes of one jj then write 8 different chunk columns
    // instead of the same banks of 8 slots that lie a multiple of 128 bytes apart)
    mb[pt] = (SJ * tt + jj) * 128 | ((((jj >> 1) & 7) ^ (F13 ? tt : 0)) << 4) | 8 * g;
  }
  for (int k = 0; k <= nsteps; ++k) {
    lds_barrier();  // the transposed rows of step k are there; the buffer of step k - 2 has been read
    // rows 2k + 4, 2k + 5 for the next step (their ring slots were last read in step k - 1; they landed before
    // barrier k: rows 4, 5 before the first one, the rest before the second); F13: the other waves do it
    if (!F13) {
      const int q = 2 * k + 4 + (wave & 1);
      if ((q & 3) == wave && q < nin) transpose_row(q, 0, 1);
    }
    const int r = 2 * k + rho;
    if (k == nsteps || r >= nout) continue;
    int rowoff[3];
#pragma unroll
    for (int dr = 0; dr < 3; ++dr) rowoff[dr] = ((r + dr) % kCvrRing) * XTROW;
    f32x16 acc[2];
#pragma unroll
    for (int pt = 0; pt < 2; ++pt)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[pt][e] = 0.f;
    constexpr int kAhead = F13 ? 5 : 3;
    V8 xf[NSTEP][2];
    auto fetch = [&](int st) __attribute__((always_inline)) {
      const int tap = st >> 2, kk = st & 3, dr = tap / 3, ds = tap - 3 * dr;
#pragma unroll
      for (int pt = 0; pt < 2; ++pt)
        xf[st][pt] = *reinterpret_cast<const V8*>(Xt + ((rowoff[dr] + xb[ds]) ^ ((2 * kk + g) << 4)) + 4096 * pt);
    };
#pragma unroll
    for (int st = 0; st < kAhead; ++st) fetch(st);
#pragma unroll
    for (int st = 0; st < NSTEP; ++st) {
      if (st + kAhead < NSTEP) fetch(st + kAhead);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int pt = 0; pt < 2; ++pt) acc[pt] = Elem<T>::mfma32(w1f[st], xf[st][pt], acc[pt]);
      __builtin_amdgcn_sched_barrier(0);
    }
    // acc[pt][4 i + e] = mid[c1 = 32 c1t + 8 i + 4 g + e][pixel]: 8 bytes into chunk 4 c1t + i of the pixel
    char* const mw = mid + (k % 3) * MIDBUF;  // (the buffers start on multiples of 128 bytes)
#pragma unroll
    for (int pt = 0; pt < 2; ++pt) {
      if (!px_ok[pt]) continue;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const V2 a0 = cvt2<T>(acc[pt][4 * i], acc[pt][4 * i + 1]), a1 = cvt2<T>(acc[pt][4 * i + 2], acc[pt][4 * i + 3]);
        V4 w = {a0[0], a0[1], a1[0], a1[1]};
        if (p.relu_mid) w = relu_packed(w);
        *reinterpret_cast<V4*>(mw + (mb[pt] ^ ((4 * c1t + i) << 4))) = w;
      }
    }
  }
#else
  (void)p;
#endif
}

template <typename T, int NI, bool F13>
hipError_t launch_conv_rows_ni(const ConvRowsArgs& args, hipStream_t stream) {
  const int lds = conv_rows_lds_bytes(args.W, args.band, F13);
  auto kern = conv_rows_kernel<T, NI, F13>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(args.N * args.bands)), dim3(64 * kCvrWaves), lds, stream, args);
  return hipGetLastError();
}

template <typename T>
hipError_t launch_conv_rows(const ConvRowsArgs& args, hipStream_t stream) {
  switch (args.W / 8) {
    case 1: return args.f13 ? launch_conv_rows_ni<T, 1, true>(args, stream)
                            : launch_conv_rows_ni<T, 1, false>(args, stream);
    case 2: return args.f13 ? launch_conv_rows_ni<T, 2, true>(args, stream)
                            : launch_conv_rows_ni<T, 2, false>(args, stream);
    case 3: return args.f13 ? launch_conv_rows_ni<T, 3, true>(args, stream)
                            : launch_conv_rows_ni<T, 3, false>(args, stream);
    case 4: return args.f13 ? launch_conv_rows_ni<T, 4, true>(args, stream)
                            : launch_conv_rows_ni<T, 4, false>(args, stream);
    case 5: return args.f13 ? launch_conv_rows_ni<T, 5, true>(args, stream)
                            : launch_conv_rows_ni<T, 5, false>(args, stream);
    case 6: return args.f13 ? launch_conv_rows_ni<T, 6, true>(args, stream)
                            : launch_conv_rows_ni<T, 6, false>(args, stream);
    case 7: return args.f13 ? launch_conv_rows_ni<T, 7, true>(args, stream)
                            : launch_conv_rows_ni<T, 7, false>(args, stream);
    case 8: return args.f13 ? launch_conv_rows_ni<T, 8, true>(args, stream)
                            : launch_conv_rows_ni<T, 8, false>(args, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace ditto
