// Fused conv(1x1) -> cast|relu -> conv(3x3, stride 1, pad 1) on NCHW tensors with at most 64 channels
// everywhere, fp16 / bf16, gfx950: persistent workgroups that keep the second convolution's weights in LDS.
//
// Reference chain: benchmark/chimera/cuda/conv1x1_conv3x3_cuda.py (the ResNet-50 row 32 x 64 x 56 x 56 ->
// 64 -> 64 of its table).  The general kernel (conv_chain.h, second convolution through LDS) streams W2
// through two small LDS buffers once per workgroup and tile: on that row six stages of 0.57 us for 0.16 us
// of MFMA each, two rounds of workgroups.  Here a workgroup of eight waves per CU loads W2 ONCE
// (9 taps x 64 x 64, 72 KB, already in MFMA fragment order) and walks over tiles of TH2 whole output rows:
//
//   X rows r0-1 .. r0+TH2 of all input channels   --direct loads-->  LDS, raw [c0][rows * W]  (one
//                                                  contiguous run per channel; rows outside the image are
//                                                  out of range and arrive as zeros)
//   first convolution, transposed (MFMA column = pixel):  mid^T[c1][px] = W1[c1][c0] . X[c0][px]
//        A = W1 fragments, resident in registers;  B = X through the transposing LDS read
//        result: a lane holds 4 consecutive c1 of one pixel per register group -> cast -> LDS mid[px][c1]
//        (128 bytes per pixel, 16-byte chunks XOR-swizzled by pixel, one zero column left and right: the
//        second convolution's padding; rows outside the image are zero because X was)
//   second convolution (MFMA row = pixel):  out[px][c2] = sum_tap mid[px + tap][c1] . W2[tap][c1][c2]
//        A = 16-byte reads of mid, B = 16-byte reads of the resident W2 fragments
//        result: with the MFMA rows dealt to the pixels in the right order a lane holds 16 consecutive pixels
//        of one output channel: 16-byte stores straight from registers, no turn-around.
//
// While the second convolution of a tile runs, the direct loads of the next tile's X rows are in flight
// (the raw X buffer is free once the first convolution is done).  Two barriers per tile.
#pragma once
#include "common.h"

namespace ditto {

struct ConvResidentArgs {
  const void* x;
  const void* w1;   // [C1][C0] as given
  const void* w2f;  // W2 in fragment order (pack_conv_w2_resident)
  void* y;
  int N, C0, H, W, C1, C2;
  int TH2;      // output rows per tile
  int tiles_h;  // tiles per image
  int ntiles;
  int relu_mid, relu_out, out_f32;
};

constexpr int kCrC = 64;  // channel extents are padded to this inside the kernel
constexpr int kCrTaps = 9;
constexpr int kCrW2Bytes = kCrTaps * (kCrC / 16) * (kCrC / 32) * 1024;  // fragments of 1 KB: [tap][k step][c2 tile]
constexpr int kCrMaxLoads = 8;                                           // direct loads of X per wave and tile

__host__ __device__ inline int conv_resident_x_bytes(int TH2, int W) { return kCrC * (TH2 + 2) * W * 2; }
__host__ __device__ inline int conv_resident_mid_bytes(int TH2, int W) { return (TH2 + 2) * (W + 2) * kCrC * 2; }
__host__ __device__ inline int conv_resident_lds_bytes(int TH2, int W) {
  return kCrW2Bytes + conv_resident_x_bytes(TH2, W) + conv_resident_mid_bytes(TH2, W);
}

// W2[c2][c1][r][s] -> [tap][c1 / 16][c2 / 32][lane][8]: lane (ln = lane % 32, g = lane / 32) of fragment
// (tap, kk, ct) holds W2[32 ct + ln][16 kk + 8 g + e][tap], e = 0..7 (zero beyond C1 / C2): the B operand
// of v_mfma_f32_32x32x16 with the output channel as column.
template <typename T>
__global__ void pack_conv_w2_resident_kernel(const T* __restrict__ w2, T* __restrict__ out, int C1, int C2) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= kCrW2Bytes / 2) return;
  const int e = i & 7, lane = (i >> 3) & 63, frag = i >> 9;
  const int ct = frag % (kCrC / 32), kk = (frag / (kCrC / 32)) % (kCrC / 16), tap = frag / ((kCrC / 32) * (kCrC / 16));
  const int c2 = 32 * ct + (lane & 31), c1 = 16 * kk + 8 * (lane >> 5) + e;
  T v = (T)0.f;
  if (c2 < C2 && c1 < C1) v = w2[((long long)c2 * C1 + c1) * kCrTaps + tap];
  out[i] = v;
}

template <typename T>
__global__ __launch_bounds__(512) void conv_chain_resident_kernel(ConvResidentArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  typedef typename Elem<T>::v2 V2;
  constexpr int NKK = kCrC / 16;  // k steps of either convolution
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int i16 = lane & 15, h = (lane >> 4) & 1;

  const int W = p.W, H = p.H, TH2 = p.TH2;
  const int MW = W + 2;                 // pixels per row of the intermediate tile
  const int rows_mid = TH2 + 2;
  const int npm = rows_mid * W;         // pixels the first convolution produces per tile
  const int npo = TH2 * W;              // output pixels per tile (<= 256)
  const int rwb = rows_mid * W * 2;     // bytes of one channel's rows in the raw X buffer
  const int xb = kCrC * rwb;
  char* const Xs = smem_raw + kCrW2Bytes;
  char* const Ms = Xs + xb;
  const unsigned lds0 = (unsigned)(size_t)(DITTO_LDS char*)smem_raw;
  const long long plane = (long long)H * W;
  const T* __restrict__ W1g = reinterpret_cast<const T*>(p.w1);
  const unsigned img_bytes = (unsigned)(p.C0 * plane * 2);

  // ---- direct loads of X: the raw buffer is [c0][rwb bytes]; load j of a wave covers 64 consecutive
  // 16-byte pieces, piece id = 64 (wave + 8 j) + lane = c0 * ppc + pc
  const int ppc = rwb / 16;
  const int nload = kCrC * ppc / 64;  // whole loads: 64 channels
  int xv[kCrMaxLoads], xrow[kCrMaxLoads];
#pragma unroll
  for (int j = 0; j < kCrMaxLoads; ++j) {
    const int id = 64 * (wave + 8 * j) + lane;
    const int c0 = id / ppc, pc = id - c0 * ppc;
    xrow[j] = c0 < p.C0 ? (pc * 8) / W : -0x10000;  // row of the piece inside the tile; never valid beyond C0
    xv[j] = (int)(c0 * plane * 2) + pc * 16;
  }
  auto load_x = [&](int tile) __attribute__((always_inline)) {
    const int n = tile / p.tiles_h, r0 = (tile - n * p.tiles_h) * TH2;
    const i32x4 rsrc = make_rsrc_uniform(reinterpret_cast<const T*>(p.x) + (long long)n * p.C0 * plane, img_bytes);
    const int shift = (r0 - 1) * W * 2;
#pragma unroll
    for (int j = 0; j < kCrMaxLoads; ++j) {
      if (wave + 8 * j < nload) {
        const int row = r0 - 1 + xrow[j];
        const unsigned vo = (row >= 0 && row < H) ? (unsigned)(xv[j] + shift) : 0x7fffffffu;
        lds_dma_16(rsrc, vo, lds0 + kCrW2Bytes + 1024 * (wave + 8 * j));
      }
    }
  };

  // ---- prologue: first X tile, W1 fragments, W2 fragments into LDS (waited for only before the first second
  // convolution), zero columns of the intermediate tile
  int tile = (int)xcd_remap(blockIdx.x, gridDim.x);
  if (tile < p.ntiles) load_x(tile);
  // A operand of the first convolution: lane (ln, g) holds W1[32 c1t + ln][16 kk + 8 g .. + 7]
  V8 w1f[2][NKK];
#pragma unroll
  for (int c1t = 0; c1t < 2; ++c1t)
#pragma unroll
    for (int kk = 0; kk < NKK; ++kk) {
      const int c1 = 32 * c1t + ln, c0 = 16 * kk + 8 * g;
      V8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (c1 < p.C1 && c0 < p.C0) v = *reinterpret_cast<const V8*>(W1g + (long long)c1 * p.C0 + c0);
      w1f[c1t][kk] = v;
    }
  constexpr int kW2Loads = kCrW2Bytes / 1024 / 8;  // per wave
  {
    const i32x4 w2_rsrc = make_rsrc(p.w2f, (unsigned)kCrW2Bytes);
#pragma unroll
    for (int j = 0; j < kW2Loads; ++j)
      lds_dma_16(w2_rsrc, (unsigned)(1024 * (wave + 8 * j) + 16 * lane), lds0 + 1024 * (wave + 8 * j));
    // pixels (row, 0) and (row, W + 1) of every row: 2 * rows_mid pixels of 128 bytes = 8 pieces of 16 each
    for (int i = tid; i < 2 * rows_mid * 8; i += 512) {
      const int px = i >> 3, row = px >> 1, col = (px & 1) ? W + 1 : 0;
      *reinterpret_cast<i32x4*>(Ms + (row * MW + col) * 128 + (i & 7) * 16) = i32x4{0, 0, 0, 0};
    }
  }

  // ---- per-lane addresses, the same for every tile
  // first convolution: pixel tile t = wave + 8 u of the intermediate tile, slot = 32 t + ln
  int x_rd[2], m_wr[2];
  bool m_ok[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int t = wave + 8 * u;
    // transposing read: lane points at channel 8 g + i16 / 4 (+ 4 for the second read), 4 pixels at 16 h + 4 (i16 % 4)
    x_rd[u] = (8 * g + (i16 >> 2)) * rwb + (32 * t + 16 * h + 4 * (i16 & 3)) * 2;
    const int slot = 32 * t + ln;
    m_ok[u] = slot < npm;
    const int mrow = slot / W, mcol = slot - mrow * W + 1;
    const int pl = mrow * MW + mcol;
    m_wr[u] = m_ok[u] ? pl * 128 + 8 * g : 0;
    // (the 16-byte chunk index of the write, 4 c1t + i, is XORed with pl & 7 at the write; a lane past the
    // tile's last pixel keeps its read address: the 16 lanes of a group transpose among themselves, and what
    // it reads lies in the next channel's run or the intermediate tile, inside LDS either way)
  }
  // second convolution: MFMA row ln = 8 i + 4 g' + e of the wave's pixel tile stands for output slot
  // 32 wave + 16 g' + 4 i + e, so that the accumulator registers of a lane (rows 8 i + 4 g + e, i and e = 0..3) are
  // 16 consecutive pixels: two 16-byte stores per lane and column tile.  Address of the lane's pixel at tap
  // (r, s), chunk XOR
  int m_rd[kCrTaps], m_x7[kCrTaps];
  {
    const int slot = 32 * wave + 16 * ((ln >> 2) & 1) + 4 * (ln >> 3) + (ln & 3);
    const int sl = slot < npo ? slot : 0;
    const int ph = sl / W, pw = sl - ph * W;
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int s = 0; s < 3; ++s) {
        const int pl = (ph + r) * MW + pw + s;
        m_rd[3 * r + s] = pl * 128;
        m_x7[3 * r + s] = (pl & 7) << 4;
      }
  }
  const int w2_rd = lane * 16;
  // output: registers 4 i + e of column tile ct hold pixels 32 wave + 16 g + 4 i + e of channel 32 ct + ln
  const int o_slot = 32 * wave + 16 * g;

  // loads return in order: the X rows (and W1) are there once only the W2 loads, issued last, are outstanding
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kW2Loads) : "memory");
  wg_sync();
  bool w2_pending = true;

  for (; tile < p.ntiles; tile += gridDim.x) {
    const int n = tile / p.tiles_h, r0 = (tile - n * p.tiles_h) * TH2;
    // ---- first convolution over the tile's rows (with halo), result to LDS; all fragments are read first
    V8 xf[2][NKK];
#pragma unroll
    for (int u = 0; u < 2; ++u)
      if (32 * (wave + 8 * u) < npm) {
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk) {
          const char* q = Xs + x_rd[u] + 16 * kk * rwb;
          V4 lo = lds_read_tr4<T>(reinterpret_cast<const T*>(q));
          V4 hi = lds_read_tr4<T>(reinterpret_cast<const T*>(q + 4 * rwb));
          xf[u][kk] = concat4<V4, V8>(lo, hi);
        }
      }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      if (32 * (wave + 8 * u) < npm) {
        f32x16 acc[2];
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
          for (int r = 0; r < 16; ++r) acc[c][r] = 0.f;
#pragma unroll
        for (int kk = 0; kk < NKK; ++kk)
#pragma unroll
          for (int c = 0; c < 2; ++c) acc[c] = Elem<T>::mfma32(w1f[c][kk], xf[u][kk], acc[c]);
        if (m_ok[u]) {
          const int x7 = (m_wr[u] >> 7) & 7;
#pragma unroll
          for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              float v0 = acc[c][4 * i], v1 = acc[c][4 * i + 1], v2 = acc[c][4 * i + 2], v3 = acc[c][4 * i + 3];
              if (p.relu_mid) { v0 = fmaxf(v0, 0.f); v1 = fmaxf(v1, 0.f); v2 = fmaxf(v2, 0.f); v3 = fmaxf(v3, 0.f); }
              const V2 a0 = cvt2<T>(v0, v1), a1 = cvt2<T>(v2, v3);
              const V4 w = {a0[0], a0[1], a1[0], a1[1]};
              *reinterpret_cast<V4*>(Ms + m_wr[u] + (((4 * c + i) ^ x7) << 4)) = w;
            }
        }
      }
    }
    if (w2_pending) {  // first tile: the W2 fragments
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      w2_pending = false;
    }
    wg_sync();  // intermediate tile complete; raw X buffer free
    if (tile + (int)gridDim.x < p.ntiles) load_x(tile + gridDim.x);

    // ---- second convolution: 32 output pixels x 64 channels per wave
    f32x16 o[2];
    if (32 * wave < npo) {
#pragma unroll
      for (int c = 0; c < 2; ++c)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[c][r] = 0.f;
      // step = (tap, k step): one fragment of the intermediate tile, two of W2, two MFMAs; fragments are
      // fetched kAhead steps before their MFMAs
      constexpr int NSTEP = kCrTaps * NKK, kAhead = 3;
      V8 mf[NSTEP], wf[NSTEP][2];
      auto fetch = [&](int st) __attribute__((always_inline)) {
        const int tap = st / NKK, kk = st % NKK;
        mf[st] = *reinterpret_cast<const V8*>(Ms + m_rd[tap] + ((((2 * kk + g) << 4)) ^ m_x7[tap]));
#pragma unroll
        for (int c = 0; c < 2; ++c) wf[st][c] = *reinterpret_cast<const V8*>(smem_raw + w2_rd + (st * 2 + c) * 1024);
      };
#pragma unroll
      for (int st = 0; st < kAhead; ++st) fetch(st);
#pragma unroll
      for (int st = 0; st < NSTEP; ++st) {
        if (st + kAhead < NSTEP) fetch(st + kAhead);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < 2; ++c) o[c] = Elem<T>::mfma32(mf[st], wf[st][c], o[c]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // The next tile's X rows (issued before this convolution) have landed, the previous tile's stores too.
    // Behind this barrier every wave is done with the intermediate tile and X is complete: the next tile's
    // first convolution may start while other waves still issue the stores below, which nobody waits for.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    if (32 * wave < npo) {
      // ---- output: 16 consecutive pixels of one channel per lane and column tile, 8 per store (fp32: 4)
      const long long y0 = (long long)n * p.C2 * plane + (long long)r0 * W;
      const int rows_left = H - r0;  // output rows of this tile inside the image
      const int lim = (rows_left < TH2 ? rows_left : TH2) * W;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const int c2 = 32 * c + ln;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
          const int s8 = o_slot + 8 * hh;  // W is a multiple of 8: the 8 pixels are in one row, inside the tile or not
          if (c2 < p.C2 && s8 < lim) {
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              v[e] = o[c][8 * hh + e];
              if (p.relu_out) v[e] = fmaxf(v[e], 0.f);
            }
            const long long off = y0 + (long long)c2 * plane + s8;
            if (p.out_f32) {
              float* dst = reinterpret_cast<float*>(p.y) + off;
              *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
              *reinterpret_cast<f32x4*>(dst + 4) = f32x4{v[4], v[5], v[6], v[7]};
            } else {
              const V2 a0 = cvt2<T>(v[0], v[1]), a1 = cvt2<T>(v[2], v[3]), a2 = cvt2<T>(v[4], v[5]), a3 = cvt2<T>(v[6], v[7]);
              const V8 w = {a0[0], a0[1], a1[0], a1[1], a2[0], a2[1], a3[0], a3[1]};
              *reinterpret_cast<V8*>(reinterpret_cast<T*>(p.y) + off) = w;
            }
          }
        }
      }
    }
  }
#else
  (void)p;
#endif
}

template <typename T>
hipError_t launch_conv_chain_resident(const ConvResidentArgs& args, int grid, hipStream_t stream) {
  const int lds = conv_resident_lds_bytes(args.TH2, args.W);
  auto kern = conv_chain_resident_kernel<T>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(512), lds, stream, args);
  return hipGetLastError();
}

template <typename T>
hipError_t pack_conv_w2_resident(const void* w2, void* out, int C1, int C2, hipStream_t stream) {
  const int total = kCrW2Bytes / 2;
  hipLaunchKernelGGL(pack_conv_w2_resident_kernel<T>, dim3((total + 255) / 256), dim3(256), 0, stream,
                     reinterpret_cast<const T*>(w2), reinterpret_cast<T*>(out), C1, C2);
  return hipGetLastError();
}

}  // namespace ditto
