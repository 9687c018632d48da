// Depthwise conv(3x3, pad 1, stride 1, one output per input channel) -> cast|relu -> conv(1x1) on NCHW
// fp16 / bf16 tensors with at most 32 input and 64 output channels and image rows of at most 128
// pixels (whole 16-byte vectors): the first separable block of a MobileNet.
//
// Reference chain: benchmark/chimera/cuda/depthwise3x3_conv1x1_small_channel_cuda.py:77-169 with
// `factor` = 1.  At that multiplier the chain is bound by memory traffic (32 channels in, 64 out per
// pixel, 9 + 64 multiply-adds per input value), so the kernel is built around the stream of image rows:
//
//  * A workgroup owns a band of output rows of one image.  ALL input rows of the band (band + 2, every
//    channel) fit in LDS, so nothing is ever overwritten: a loader wave that does nothing else issues
//    them as direct global -> LDS loads ([channel][W] per row, 1 KB per instruction; rows above and
//    below the image are out of range and arrive as zeros) as fast as the outstanding-load counter
//    allows, and only waits for the row the compute waves need next.  It issues no stores, so its
//    counter waits are exact; the compute waves issue no loads, so nobody ever waits for a store.
//  * Depthwise stage, one output row per step: lane = (channel, strip of 8 pixels).  The lane keeps
//    the strip's three input rows in registers (10 values each) and reads only the new row per step,
//    one step ahead; 8 pixels x 3 rows x (one v_dot2 + one multiply-add) in fp32; the cast row goes to
//    LDS as mid[pixel][32 channels] (16-byte chunks XOR-swizzled by pixel group, double buffered).
//  * 1x1 stage of the previous row, same step, on four waves of their own (16 output channels each,
//    W2 fragment resident in registers): out^T[c2][pixel] = W2[c2][:] . mid[pixel][:] is ONE 16x16x32
//    MFMA per 16 output channels x 16 pixels.  MFMA column j of tile t is pixel 8 j + t, so after the
//    eight tiles of a row a lane holds 8 consecutive pixels of each of its 4 channels and the 16 lanes
//    of a column group write 256 contiguous bytes of a channel with one 16-byte store each, no
//    turn-around.  (Stores whose neighbouring lanes hit different 128-byte lines run at half the
//    device's write bandwidth; waves that wait in the store queue do nothing else here.)
//  One barrier per output row.
//
// Non-finite inputs behave as in the reference (every product is of values inside the 3x3 window).
#pragma once
#include "common.h"

namespace ditto {

struct DwRowsArgs {
  const void* x;   // [N][C0][H][W]
  const void* w1;  // [C0][1][3][3]
  const void* w2;  // [C2][C0]
  void* y;         // [N][C2][H][W]
  int N, C0, H, W, C2;
  int band, bands;  // output rows per workgroup, workgroups per image
  int relu_mid, relu_out;
};

constexpr int kDwRowsC = 32;        // input channels (padded)
constexpr int kDwRowsWaves = 13;    // eight depthwise waves, four 1x1 / store waves, the loader
constexpr int kDwRowsMaxAhead = 12; // input rows the loader keeps in flight at most

__host__ __device__ constexpr int dw_rows_ni(int W) { return (W + 15) / 16; }
// LDS: 16 bytes, band + 2 row slots of NI KB, 16 bytes, two intermediate rows of 128 pixel slots of 64 bytes
__host__ __device__ constexpr int dw_rows_lds_bytes(int W, int band) {
  return 32 + (band + 2) * 1024 * dw_rows_ni(W) + 2 * 128 * 64;
}

// wait until at most k rows of NI load instructions each are outstanding
template <int NI>
__device__ __forceinline__ void dw_rows_wait(int k) {
#define DITTO_DWR_CASE(K)                                                          \
  case K:                                                                          \
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NI * K <= 63 ? NI * K : 63) : "memory"); \
    break;
  switch (k) {
    DITTO_DWR_CASE(1)
    DITTO_DWR_CASE(2)
    DITTO_DWR_CASE(3)
    DITTO_DWR_CASE(4)
    DITTO_DWR_CASE(5)
    DITTO_DWR_CASE(6)
    DITTO_DWR_CASE(7)
    DITTO_DWR_CASE(8)
    DITTO_DWR_CASE(9)
    DITTO_DWR_CASE(10)
    DITTO_DWR_CASE(11)
    default:
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
#undef DITTO_DWR_CASE
}

template <typename T, int NI>
__global__ __launch_bounds__(64 * kDwRowsWaves) void dw_rows_kernel(DwRowsArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v2 V2;
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  constexpr int SLOT = 1024 * NI;
  constexpr unsigned kOut = 0x7fffffffu;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int W = p.W, H = p.H, S = W >> 3;
  const unsigned wg = xcd_remap(blockIdx.x, gridDim.x);
  const int n = (int)wg / p.bands, y0 = ((int)wg - n * p.bands) * p.band;
  const int nout = H - y0 < p.band ? H - y0 : p.band;  // output rows of this band
  const int nin = nout + 2;                            // input rows y0 - 1 .. y0 + nout
  const long long plane = (long long)H * W;
  char* const rows = smem_raw + 16;
  char* const mids = rows + (p.band + 2) * SLOT + 16;
  const unsigned lds0 = (unsigned)(size_t)(DITTO_LDS char*)smem_raw;

  if (wave == 12) {
    // ======================= loader wave =======================
    // instruction i of a row: lane l brings 16 bytes of job 64 i + l = channel * S + strip
    const i32x4 rsrc = make_rsrc_uniform(reinterpret_cast<const T*>(p.x) + (long long)n * p.C0 * plane,
                                         (unsigned)(p.C0 * plane * 2));
    unsigned vo[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int job = 64 * i + lane, c = job / S, strip = job - c * S;
      vo[i] = c < kDwRowsC ? (unsigned)(c * (int)plane * 2 + strip * 16) : kOut;  // channels >= C0 are out of range
    }
    auto issue = [&](int k) __attribute__((always_inline)) {
      const int y = y0 - 1 + k;
      const bool ok = y >= 0 && y < H;
      const unsigned shift = (unsigned)(y * W * 2);
#pragma unroll
      for (int i = 0; i < NI; ++i) lds_dma_16(rsrc, ok ? vo[i] + shift : kOut, lds0 + 16 + k * SLOT + 1024 * i);
    };
    constexpr int AH = 63 / NI < kDwRowsMaxAhead ? 63 / NI : kDwRowsMaxAhead;
    int issued = 0;
    while (issued < nin && issued < AH) issue(issued++);
    dw_rows_wait<NI>(issued - 3 > 0 ? issued - 3 : 0);  // input rows 0, 1, 2: what the depthwise waves start from
    lds_barrier();
    for (int r = 0; r <= nout; ++r) {
      // the compute waves read input row r + 3 during step r (one step ahead of its use)
      const int need = r + 3 < nin - 1 ? r + 3 : nin - 1;
      int k = issued - 1 - need;  // rows that may still be outstanding
      if (k < 0) k = 0;
      dw_rows_wait<NI>(k);
      lds_barrier();
      while (issued < nin && k < AH) {
        issue(issued++);
        ++k;
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    return;
  }

  if (wave >= 8) {
    // ======================= 1x1 / store waves =======================
    const int c2q = wave - 8;
    const int j = lane & 15, kg = lane >> 4;
    // A operand: lane (m, kg) holds W2[16 c2q + m][8 kg .. + 7]
    V8 wf;
    {
      const T* W2g = reinterpret_cast<const T*>(p.w2);
      const int c2 = 16 * c2q + j;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int ch = 8 * kg + e;
        wf[e] = (c2 < p.C2 && ch < p.C0) ? W2g[(long long)c2 * p.C0 + ch] : (T)0.f;
      }
    }
    // B operand of tile t: lane (j, kg) reads channels 8 kg .. + 7 of pixel 8 j + t (slot 16 t + j)
    const int b_rd = 64 * j + 16 * (kg ^ ((j >> 2) & 3));
    // result: register i of tile t is out[c2 = 16 c2q + 4 kg + i][pixel 8 j + t]
    unsigned y_vo[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c2 = 16 * c2q + 4 * kg + i;
      y_vo[i] = (c2 < p.C2 && 8 * j < W) ? (unsigned)(c2 * (int)plane * 2 + 16 * j) : kOut;
    }
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        reinterpret_cast<T*>(p.y) + (long long)n * p.C2 * plane, 0, (int)(p.C2 * plane * 2), 0x00020000);
    lds_barrier();
    for (int r = 0; r <= nout; ++r) {
      lds_barrier();  // mid row r - 1 is written
      if (r == 0) continue;
      const char* const mr = mids + ((r - 1) & 1) * (128 * 64) + b_rd;
      V8 bf[8];
#pragma unroll
      for (int t = 0; t < 8; ++t) bf[t] = *reinterpret_cast<const V8*>(mr + 1024 * t);
      f32x4 o[8];
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < 8; ++t) o[t] = Elem<T>::mfma16(wf, bf[t], z);
      const unsigned soff = (unsigned)((y0 + r - 1) * W * 2);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v[8];
#pragma unroll
        for (int t = 0; t < 8; ++t) v[t] = p.relu_out ? fmaxf(o[t][i], 0.f) : o[t][i];
        const V2 q0 = cvt2<T>(v[0], v[1]), q1 = cvt2<T>(v[2], v[3]), q2 = cvt2<T>(v[4], v[5]), q3 = cvt2<T>(v[6], v[7]);
        const V8 px8 = {q0[0], q0[1], q1[0], q1[1], q2[0], q2[1], q3[0], q3[1]};
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, px8), y_rsrc, y_vo[i], soff, kStoreWriteThrough);
      }
    }
    return;
  }

  // ======================= depthwise waves =======================
  // job = (channel c, strip of 8 pixels)
  const int job = 64 * wave + lane;
  const bool dw_wave = wave < NI;  // wave-uniform
  const int c = job / S, strip = job - c * S;
  const bool dw_on = c < kDwRowsC;
  V2 w01[3], w12[3];
  float w0f[3], w2f[3];
  {
    const T* W1g = reinterpret_cast<const T*>(p.w1);
    const T zero = (T)0.f;
#pragma unroll
    for (int rr = 0; rr < 3; ++rr) {
      T a = zero, b = zero, d = zero;
      if (dw_wave && c < p.C0) {
        a = W1g[c * 9 + 3 * rr];
        b = W1g[c * 9 + 3 * rr + 1];
        d = W1g[c * 9 + 3 * rr + 2];
      }
      w01[rr] = V2{a, b};
      w12[rr] = V2{b, d};
      w0f[rr] = (float)a;
      w2f[rr] = (float)d;
    }
  }
  const bool first_strip = strip == 0, last_strip = strip == S - 1;
  // a strip's row: the dword left of it (its high half is pixel -1), its own four dwords, the dword right of it
  struct Row {
    unsigned l, d[4], r;
  };
  auto read_row = [&](int slot) __attribute__((always_inline)) -> Row {
    const char* q = rows + slot * SLOT + job * 16;
    Row v;
    const u32x4 own = *reinterpret_cast<const u32x4*>(q);
    v.l = *reinterpret_cast<const unsigned*>(q - 4);
    v.r = *reinterpret_cast<const unsigned*>(q + 16);
    v.d[0] = own[0]; v.d[1] = own[1]; v.d[2] = own[2]; v.d[3] = own[3];
    if (first_strip) v.l = 0;  // the image's zero padding
    if (last_strip) v.r = 0;
    return v;
  };
  auto lo = [](unsigned d) __attribute__((always_inline)) { return (float)__builtin_bit_cast(V2, d)[0]; };
  auto hi = [](unsigned d) __attribute__((always_inline)) { return (float)__builtin_bit_cast(V2, d)[1]; };
  auto dw_accumulate = [&](const Row& v, int rr, float* acc) __attribute__((always_inline)) {
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      const V2 dm = __builtin_bit_cast(V2, v.d[m]);
      // pixel 2m: values 2m-1, 2m, 2m+1;  pixel 2m+1: values 2m, 2m+1, 2m+2
      acc[2 * m] = Elem<T>::dot2(dm, w12[rr], fmaf(hi(m ? v.d[m - 1] : v.l), w0f[rr], acc[2 * m]));
      acc[2 * m + 1] = Elem<T>::dot2(dm, w01[rr], fmaf(lo(m < 3 ? v.d[m + 1] : v.r), w2f[rr], acc[2 * m + 1]));
    }
  };
  // intermediate row: pixel 8 j + t lives in slot 16 t + j (64 bytes: 32 channels), its 16-byte chunk ch at
  // chunk ch ^ ((j >> 2) & 3): the 16 lanes of an MFMA operand read (fixed t, j = 0..15) hit every bank once
  const int mid_wr = 64 * strip + 16 * ((c >> 3) ^ ((strip >> 2) & 3)) + 2 * (c & 7);

  Row r0, r1, r2, nx;
  lds_barrier();  // input rows 0, 1, 2 have landed
  if (dw_wave) {
    r1 = read_row(0);
    r2 = read_row(1);
    nx = read_row(2);
  }
  for (int r = 0; r <= nout; ++r) {
    lds_barrier();  // input rows <= r + 3 have landed; mid row r - 2 has been consumed
    if (dw_wave && r < nout) {
      r0 = r1;
      r1 = r2;
      r2 = nx;
      if (r + 3 < nin) nx = read_row(r + 3);
      float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      dw_accumulate(r0, 0, acc);
      dw_accumulate(r1, 1, acc);
      dw_accumulate(r2, 2, acc);
      if (dw_on) {
        T* const mw = reinterpret_cast<T*>(mids + (r & 1) * (128 * 64) + mid_wr);
#pragma unroll
        for (int i = 0; i < 8; ++i) mw[512 * i] = (T)(p.relu_mid ? fmaxf(acc[i], 0.f) : acc[i]);
      }
    }
  }
#else
  (void)p;
#endif
}

template <typename T, int NI>
hipError_t launch_dw_rows_ni(const DwRowsArgs& args, hipStream_t stream) {
  const int lds = dw_rows_lds_bytes(args.W, args.band);
  auto kern = dw_rows_kernel<T, NI>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  hipLaunchKernelGGL(kern, dim3((unsigned)(args.N * args.bands)), dim3(64 * kDwRowsWaves), lds, stream, args);
  return hipGetLastError();
}

template <typename T>
hipError_t launch_dw_rows(const DwRowsArgs& args, hipStream_t stream) {
  switch (dw_rows_ni(args.W)) {
    case 1: return launch_dw_rows_ni<T, 1>(args, stream);
    case 2: return launch_dw_rows_ni<T, 2>(args, stream);
    case 3: return launch_dw_rows_ni<T, 3>(args, stream);
    case 4: return launch_dw_rows_ni<T, 4>(args, stream);
    case 5: return launch_dw_rows_ni<T, 5>(args, stream);
    case 6: return launch_dw_rows_ni<T, 6>(args, stream);
    case 7: return launch_dw_rows_ni<T, 7>(args, stream);
    case 8: return launch_dw_rows_ni<T, 8>(args, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace ditto
