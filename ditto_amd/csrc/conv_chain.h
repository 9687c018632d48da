// Fused conv(RxS) -> cast|relu -> conv(1x1) chain on NCHW tensors, fp16 / bf16, gfx950.
//
// Reference chain: benchmark/chimera/cuda/conv3x3_conv1x1_cuda.py:77-172 (conv -> cast ->
// conv, fp32 accumulate), ReLU variant conv_relu_conv_relu_fuse_hw_cuda.py:134-142 (ReLU on
// the accumulator, then cast).  The reference takes pre-padded images and weights packed
// in 16-channel blocks; here the plain NCHW / KCRS tensors are consumed directly and
// re-laid out while they are staged into LDS.
//
// Both convolutions are computed TRANSPOSED as implicit GEMMs whose MFMA column index is
// the output pixel:
//     mid^T[c1][pix] = sum_{r,s,c0} W1[c1][c0][r][s] * X[c0][pix shifted by (r,s)]
//     out^T[c2][pix] = sum_{c1}     W2[c2][c1]       * cast(mid^T[c1][pix])
// so the accumulator registers of the first (lane = pixel, 16 channels per 32x32 tile) are,
// after the cast, exactly the B operand of the second: the intermediate feature map never
// leaves VGPRs, and a lane's results for one output channel are consecutive pixels, i.e.
// contiguous in NCHW.
//
// A workgroup (4 waves) owns TH output rows x TW output columns of one image
// (TH*TW <= 128*PXW pixel slots, 32*PXW per wave) and all C1 / C2 channels.  Input channels
// are walked in chunks of 32: the halo tile X[32][rows_in][cols_in] is staged to LDS as
// [row][col][channel] and the weight chunk as [r*S+s][c1][channel], so that both MFMA
// operands are 16-byte LDS reads.  W2 is staged row by row through the same LDS once the first
// convolution is done.  The tile is sized so that two workgroups fit in a CU's LDS: one
// stages while the other feeds the MFMA pipe.
#pragma once
#include <type_traits>

#include "common.h"

namespace ditto {

struct ConvChainArgs {
  const void* x;
  const void* w1;
  const void* w2;
  const void* w1p;   // W1 repacked by pack_conv_w1 (null: the kernel re-lays W1 out itself, slower)
  void* y;
  int N, C0, H, W;
  int C1, R, S, pad, stride;
  int C2;
  int P, Q;          // output extent of both convolutions (conv2 is 1x1, stride 1)
  int TH, TW;        // output tile per workgroup
  int tiles_h, tiles_w;
  int rows_in, cols_in;  // halo tile extent
  int relu_mid, relu_out, out_f32;
  // second convolution larger than 1x1: then P, Q, TH, TW above describe the
  // INTERMEDIATE tile (the output tile grown by the second filter's halo) and these the output
  const void* w2p;   // W2 repacked by pack_conv_w2
  int R2, S2, pad2;
  int P2, Q2;        // output extent
  int TH2, TW2;      // output tile per workgroup
  int wide2;         // 16-byte output stores through LDS: Q2 and TW2 multiples of 8, y 16-byte aligned, not fp32
  int stride2;       // stride of the second convolution (the 1x1 second convolution is always run with stride 1)
};

// Input channels per staged chunk: 32 (two MFMA k steps per tap) or, where that does not fit in
// LDS, 16.  A channel vector is padded by 8 elements in LDS (strides of 80 / 48 bytes put the
// 16-byte reads of consecutive pixels / rows into different bank groups).
__host__ __device__ constexpr int conv_ch_stride(int ch) { return ch + 8; }

// bytes of one repacked W1 chunk [R*S][C1p][ch + 8]
__host__ __device__ inline int conv_w1_chunk_bytes(int RS, int C1p, int ch) { return RS * C1p * conv_ch_stride(ch) * 2; }

__host__ __device__ inline int conv_chain_lds_bytes(int rows_in, int cols_in, int RS, int C1p, int ch) {
  // halo tile, then the W1 chunk rounded up to whole 1 KB direct-load instructions
  const int first = rows_in * cols_in * conv_ch_stride(ch) * 2 + (conv_w1_chunk_bytes(RS, C1p, ch) + 1023) / 1024 * 1024;
  const int second = 32 * (C1p + 4) * 2;  // at least 32 rows of W2
  return first > second ? first : second;
}

// Second convolution larger than 1x1: the intermediate tile lives in LDS as [slot][C1p + 8] and W2
// streams through two buffers of [S2][64 output channels][32 + 8]: one filter row of a chunk of 32
// intermediate channels for a block of 64 output channels per stage (small enough for two
// workgroups per CU).  The packed W2 holds the R2 rows of a (block, chunk) back to back.  `wide`
// adds the per-wave turn-around buffers of the 16-byte output stores.
constexpr int kConv2Oss = 40;  // row stride (elements) of a wave's output turn-around buffer: 32 pixels + 8
__host__ __device__ inline int conv_w2_chunk_bytes(int RS2) { return RS2 * 64 * conv_ch_stride(32) * 2; }
__host__ __device__ inline int conv_w2_row_bytes(int S2) { return S2 * 64 * conv_ch_stride(32) * 2; }
__host__ __device__ inline int conv_chain2_lds_bytes(int slots, int C1p, int S2, bool wide) {
  return slots * (C1p + 8) * 2 + 2 * ((conv_w2_row_bytes(S2) + 1023) / 1024 * 1024) + (wide ? 4 * 32 * kConv2Oss * 2 : 0);
}

// The packed W2 is [c2 / 64][c1 / 32][r*S2+s][64][32 + 8] (zero padded); see pack_conv_w12_kernel.

// W1[c1][c0][r][s] -> chunks [c0 / ch][r*S+s][C1p][ch + 8] (zero padded): the layout the chain
// kernel keeps a chunk in, so that it can load one with direct global -> LDS copies.
template <typename T>
__global__ void pack_conv_w1_kernel(const T* __restrict__ w1, T* __restrict__ out, int C0, int C1, int RS, int C1p, int ch,
                                    long long total) {
  const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;  // the packed tensors are far below 2^31 elements
  if (i >= total) return;
  const unsigned chs = conv_ch_stride(ch);
  const int c = (int)(i % chs);
  unsigned q = i / chs;
  const int c1 = (int)(q % (unsigned)C1p);
  q /= (unsigned)C1p;
  const int rs = (int)(q % (unsigned)RS);
  const int chunk = (int)(q / (unsigned)RS);
  const int c0 = chunk * ch + c;
  T v = (T)0.f;
  if (c < ch && c1 < C1 && c0 < C0) v = w1[((long long)c1 * C0 + c0) * RS + rs];
  out[i] = v;
}

// PX2 = 0: the second convolution is 1x1 and consumes the first one's accumulators from registers;
// PX2 = 1 | 2: it is R2 x S2 (any stride) and reads the intermediate tile from LDS, PX2 tiles of 32
// output pixels per wave.
template <typename T, int C1T, int PXW, int CH, int PX2 = 0>
__global__ __launch_bounds__(256) void conv_chain_kernel(ConvChainArgs p) {
#if defined(__HIP_DEVICE_COMPILE__)
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  constexpr int C1p = 32 * C1T;
  constexpr int CHS = conv_ch_stride(CH);
  constexpr int W2S = C1p + 4;  // LDS row stride of the staged W2 block (8-byte reads, conflict-free)
  extern __shared__ __attribute__((aligned(1024))) char smem_raw[];
  T* const Xs = reinterpret_cast<T*>(smem_raw);                // [rows_in][cols_in][CHS]
  T* const Ws = Xs + p.rows_in * p.cols_in * CHS;              // [R*S][C1p][CHS]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ln = lane & 31, g = lane >> 5;
  const int RS = p.R * p.S;

  // workgroup -> (image, tile row, tile column); neighbouring ids share an image
  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
  const int tiles = p.tiles_h * p.tiles_w;
  const int n = lid / tiles;
  const int th = (lid % tiles) / p.tiles_w, tw = (lid % tiles) % p.tiles_w;
  // origin of the tile the FIRST convolution produces (the intermediate tile when PX2 > 0)
  const int p0 = PX2 ? th * p.TH2 * p.stride2 - p.pad2 : th * p.TH, q0 = PX2 ? tw * p.TW2 * p.stride2 - p.pad2 : tw * p.TW;
  const int h0 = p0 * p.stride - p.pad, w0 = q0 * p.stride - p.pad;  // input coords of the halo origin

  const T* __restrict__ Xg = reinterpret_cast<const T*>(p.x) + (long long)n * p.C0 * p.H * p.W;
  const T* __restrict__ W1g = reinterpret_cast<const T*>(p.w1);
  const T* __restrict__ W2g = reinterpret_cast<const T*>(p.w2);

  // pixel slots of this lane: slot = 32*(PXW*wave + j) + ln  ->  (ph, pw) inside the tile
  int xoff[PXW];   // LDS element offset of the lane's pixel at (r,s) = (0,0)
  bool valid[PXW];
  int opix[PXW];   // offset of the pixel inside one output channel plane
#pragma unroll
  for (int j = 0; j < PXW; ++j) {
    const int slot = 32 * (PXW * wave + j) + ln;
    const int ph = slot / p.TW, pw = slot % p.TW;
    valid[j] = ph < p.TH && (p0 + ph) >= 0 && (p0 + ph) < p.P && (q0 + pw) >= 0 && (q0 + pw) < p.Q;
    const int phc = valid[j] ? ph : 0, pwc = valid[j] ? pw : 0;
    xoff[j] = ((phc * p.stride) * p.cols_in + pwc * p.stride) * CHS + 8 * g;
    opix[j] = (p0 + phc) * p.Q + q0 + pwc;
  }

  f32x16 acc[C1T][PXW];
#pragma unroll
  for (int c = 0; c < C1T; ++c)
#pragma unroll
    for (int j = 0; j < PXW; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[c][j][r] = 0.f;

  const T zero = (T)0.f;
  const long long hw = (long long)p.H * p.W;
  // in-kernel W1 staging (no repacked copy given) walks, for one c1, the contiguous run of CH*RS
  // source elements 64 at a time; a lane's element index advances by 64 per step, i.e. its
  // (channel, tap) pair by (dq, dr)
  const int dq = 64 / RS, dr = 64 % RS;
  const int c_first = lane / RS, rs_first = lane % RS;
  const int wrun = CH * RS;
  // repacked W1: one chunk is w1_bytes contiguous bytes, copied by 1 KB direct loads
  const int w1_bytes = conv_w1_chunk_bytes(RS, C1p, CH);
  const int nchunks = (p.C0 + CH - 1) / CH;
  const i32x4 w1_rsrc = make_rsrc(p.w1p, (unsigned)(w1_bytes * nchunks));
  const unsigned ws_lds = (unsigned)(size_t)(DITTO_LDS char*)smem_raw + p.rows_in * p.cols_in * CHS * 2;

  // ---- set-up of the second convolution (1x1).  W2 is staged through the LDS the first
  // convolution has finished with, as many rows (output channels) at a time as fit, rows zero-padded to C1p.
  const long long plane = (long long)p.P * p.Q;
  const bool y_small = (long long)p.C2 * plane * 2 < 0x7fffffffLL;  // an image's output within a 32-bit buffer offset
  T* const W2s = reinterpret_cast<T*>(smem_raw);
  const int lds_elems = conv_chain_lds_bytes(p.rows_in, p.cols_in, RS, C1p, CH) / 2;
  // Output path.  A lane holds ONE pixel per register, so storing from registers means 2-byte
  // stores.  When the tile is a run of whole image rows (its pixels are contiguous in a channel
  // plane) and everything is 16-byte aligned, each wave instead turns its 32-channel x 32*PXW
  // pixel result around in a private corner of LDS and stores 8 pixels (16 bytes) per lane.
  constexpr int SLW = 32 * PXW;          // pixel slots of a wave
  constexpr int OSS = SLW + 8;           // LDS row stride of the turn-around buffer (elements)
  constexpr int OS_ELEMS = 4 * 32 * OSS; // four waves
  const int nvalid = (p.P - p0 < p.TH ? p.P - p0 : p.TH) * p.Q;  // valid slots when TW == Q
  const bool wide = p.TW == p.Q && !p.out_f32 && (nvalid & 7) == 0 && ((p0 * p.Q) & 7) == 0 && (plane & 7) == 0 &&
              (reinterpret_cast<unsigned long long>(p.y) & 15) == 0 && lds_elems - OS_ELEMS >= 32 * W2S;
  int c2blk = ((wide ? lds_elems - OS_ELEMS : lds_elems) / W2S) & ~31;
  if (c2blk > ((p.C2 + 31) & ~31)) c2blk = (p.C2 + 31) & ~31;
  T* const Os = W2s + (lds_elems - OS_ELEMS) + wave * 32 * OSS;  // this wave's turn-around buffer
  constexpr int VPR = C1p / 8;  // 16-byte vectors per staged row
  // The first W2 block is fetched into the halo-tile staging registers during the MFMAs of the
  // last chunk (they are free by then) when it is at most 8 vectors per thread.
  const bool w2_prefetch = c2blk * VPR <= 8 * 256;
  auto w2_load = [&](int cb, int e) __attribute__((always_inline)) -> i32x4 {
    const int row = e / VPR, vc = e % VPR;
    i32x4 v = {0, 0, 0, 0};
    if (e < c2blk * VPR && cb + row < p.C2 && 8 * vc < p.C1)
      v = *reinterpret_cast<const i32x4*>(W2g + (long long)(cb + row) * p.C1 + 8 * vc);
    return v;
  };
  auto w2_store = [&](int e, i32x4 v) __attribute__((always_inline)) {
    const int row = e / VPR, vc = e % VPR;
    if (e < c2blk * VPR) {  // rows are only 8-byte aligned
      *reinterpret_cast<i32x2*>(W2s + row * W2S + 8 * vc) = i32x2{v[0], v[1]};
      *reinterpret_cast<i32x2*>(W2s + row * W2S + 8 * vc + 4) = i32x2{v[2], v[3]};
    }
  };

  // ---- halo tile staging: X[c0..c0+CH-1][halo] goes to LDS as [row][col][channel].
  // Two-byte global loads issue very slowly, so when the image rows are 16-byte multiples a task
  // is an aligned group of 8 pixels x 8 channels of one halo row: eight 16-byte loads (one per
  // channel), an 8x8 transposition in registers (one byte-permute per output dword) and eight
  // 16-byte LDS writes (one per pixel).  If every thread has at most one task per chunk, the
  // loads of chunk i+1 are issued before the MFMAs of chunk i and written to LDS after them.
  const bool x_vec = (p.W & 7) == 0 && (reinterpret_cast<unsigned long long>(p.x) & 15) == 0;
  const int wg0 = (w0 >= 0 ? w0 : w0 - 7) / 8 * 8;              // first aligned group (floor)
  const int ngc = (w0 + p.cols_in - wg0 + 7) / 8;               // groups per halo row
  const int xtasks = p.rows_in * ngc * (CH / 8);
  const bool x_prefetch = x_vec && xtasks <= 256;
  // task of this thread: channel group fastest, then column group, then row
  const int t_chg = tid % (CH / 8), t_gi = (tid / (CH / 8)) % ngc, t_ri = tid / (CH / 8) / ngc;
  i32x4 xr[8];
  auto xv_load = [&](int c0, int chg, int gi, int ri, bool live) __attribute__((always_inline)) {
    const int h = h0 + ri, wg = wg0 + 8 * gi;
    const bool ok = live && h >= 0 && h < p.H && wg >= 0 && wg < p.W;
    const T* src = Xg + (long long)(c0 + 8 * chg) * hw + (long long)h * p.W + wg;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      i32x4 v = {0, 0, 0, 0};
      if (ok && c0 + 8 * chg + c < p.C0) v = *reinterpret_cast<const i32x4*>(src + c * hw);
      xr[c] = v;
    }
  };
  auto xv_store = [&](int chg, int gi, int ri, bool live) __attribute__((always_inline)) {
    const int ci0 = wg0 + 8 * gi - w0;  // halo column of the group's first pixel
#pragma unroll
    for (int px = 0; px < 8; ++px) {
      i32x4 o;
#pragma unroll
      for (int d = 0; d < 4; ++d)
        o[d] = __builtin_amdgcn_perm(xr[2 * d + 1][px >> 1], xr[2 * d][px >> 1], (px & 1) ? 0x07060302 : 0x05040100);
      const int ci = ci0 + px;
      if (live && ci >= 0 && ci < p.cols_in)
        *reinterpret_cast<i32x4*>(Xs + (ri * p.cols_in + ci) * CHS + 8 * chg) = o;
    }
  };
  if (x_prefetch) xv_load(0, t_chg, t_gi, t_ri, tid < xtasks);

  for (int c0 = 0, chunk = 0; c0 < p.C0; c0 += CH, ++chunk) {
    wg_sync();  // everyone is done reading the previous chunk
    if (p.w1p) {
      // the W1 chunk streams into LDS while the halo tile is staged through registers below
      for (int j = wave; j * 1024 < w1_bytes; j += 4) {
        const int off = j * 1024 + lane * 16;
        lds_dma_16(w1_rsrc, off < w1_bytes ? (unsigned)(chunk * w1_bytes + off) : 0x7fffffffu, ws_lds + j * 1024);
      }
    }
    if (x_prefetch) {
      xv_store(t_chg, t_gi, t_ri, tid < xtasks);
    } else if (x_vec) {
      for (int t = tid; t < xtasks; t += 256) {
        const int chg = t % (CH / 8), gi = (t / (CH / 8)) % ngc, ri = t / (CH / 8) / ngc;
        xv_load(c0, chg, gi, ri, true);
        xv_store(chg, gi, ri, true);
      }
    } else {
      // rows that are not 16-byte multiples: a lane owns one halo column and, per task, one
      // (row, group of 4 channels): four 2-byte loads, one 8-byte LDS write; four tasks in flight
      constexpr int CG = CH / 4;
      for (int rc0 = wave; rc0 < CG * p.rows_in; rc0 += 16) {
        for (int ci = lane; ci < p.cols_in; ci += 64) {
          const int w = w0 + ci;
          const bool col_ok = w >= 0 && w < p.W;
          V4 v[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int rc = rc0 + 4 * t;
            const int cg = rc & (CG - 1), ri = rc / CG;
            const int h = h0 + ri;
            const bool ok = col_ok && rc < CG * p.rows_in && h >= 0 && h < p.H;
            const T* src = Xg + (long long)(c0 + 4 * cg) * hw + (long long)h * p.W + w;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[t][e] = (ok && c0 + 4 * cg + e < p.C0) ? src[e * hw] : zero;
          }
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int rc = rc0 + 4 * t;
            const int cg = rc & (CG - 1), ri = rc / CG;
            if (rc < CG * p.rows_in) *reinterpret_cast<V4*>(Xs + (ri * p.cols_in + ci) * CHS + 4 * cg) = v[t];
          }
        }
      }
    }
    if (!p.w1p) {
      // ---- stage W1[c1][c0..c0+CH-1][r][s] as [r*S+s][c1][channel]; for one c1 the CH*RS source
      //      elements are contiguous and consecutive lanes read consecutive elements
      for (int c1 = wave; c1 < C1p; c1 += 4) {
        const T* src = W1g + ((long long)c1 * p.C0 + c0) * RS;
        int c = c_first, rs = rs_first;
        for (int e = lane; e < wrun; e += 64) {
          T v = zero;
          if (c1 < p.C1 && c0 + c < p.C0) v = src[e];
          Ws[(rs * C1p + c1) * CHS + c] = v;
          c += dq;
          rs += dr;
          if (rs >= RS) rs -= RS, ++c;
        }
      }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    wg_sync();
    if (x_prefetch && c0 + CH < p.C0) xv_load(c0 + CH, t_chg, t_gi, t_ri, tid < xtasks);  // in flight during the MFMAs
    if (PX2 == 0 && w2_prefetch && c0 + CH >= p.C0) {
#pragma unroll
      for (int k = 0; k < 8; ++k) xr[k] = w2_load(0, tid + 256 * k);
    }
    // ---- first convolution: CH/16 MFMA k steps per filter tap
    for (int r = 0; r < p.R; ++r)
      for (int s = 0; s < p.S; ++s) {
        const int tap = (r * p.cols_in + s) * CHS;
        const T* wrow = Ws + ((r * p.S + s) * C1p + ln) * CHS + 8 * g;
        V8 xf[CH / 16][PXW], wf[CH / 16][C1T];
#pragma unroll
        for (int kk = 0; kk < CH / 16; ++kk) {
#pragma unroll
          for (int j = 0; j < PXW; ++j) xf[kk][j] = *reinterpret_cast<const V8*>(Xs + xoff[j] + tap + 16 * kk);
#pragma unroll
          for (int c = 0; c < C1T; ++c) wf[kk][c] = *reinterpret_cast<const V8*>(wrow + 32 * c * CHS + 16 * kk);
        }
#pragma unroll
        for (int kk = 0; kk < CH / 16; ++kk)
#pragma unroll
          for (int c = 0; c < C1T; ++c)
#pragma unroll
            for (int j = 0; j < PXW; ++j) acc[c][j] = Elem<T>::mfma32(wf[kk][c], xf[kk][j], acc[c][j]);
      }
  }

  if constexpr (PX2 > 0) {
    // ================= second convolution R2 x S2, intermediate tile through LDS =================
    constexpr int MS = C1p + 8;  // element stride of an intermediate pixel's channel vector
    T* const Ms = reinterpret_cast<T*>(smem_raw);  // [128*PXW][MS]
    T* const W2b = Ms + 128 * PXW * MS;            // two row-chunk buffers
    const int RS2 = p.R2 * p.S2;
    const int w2_bytes = conv_w2_row_bytes(p.S2);
    const int w2_buf = (w2_bytes + 1023) / 1024 * 1024;
    constexpr int nch2 = C1p / 32;
    const int nc2b = (p.C2 + 63) / 64;
    const int nstage = nc2b * nch2 * p.R2;  // stage = (output block, intermediate chunk, filter row)
    const i32x4 w2_rsrc = make_rsrc(p.w2p, (unsigned)(w2_bytes * nstage));
    const unsigned w2_lds = (unsigned)(size_t)(DITTO_LDS char*)smem_raw + 128 * PXW * MS * 2;
    T* const Ow = reinterpret_cast<T*>(reinterpret_cast<char*>(W2b) + 2 * w2_buf) + wave * 32 * kConv2Oss;
    auto w2_issue = [&](int stage) __attribute__((always_inline)) {
      for (int j = wave; j * 1024 < w2_bytes; j += 4) {
        const int off = j * 1024 + lane * 16;
        lds_dma_16(w2_rsrc, off < w2_bytes ? (unsigned)(stage * w2_bytes + off) : 0x7fffffffu,
                   w2_lds + (stage & 1) * w2_buf + j * 1024);
      }
    };
    wg_sync();  // the first convolution's LDS is no longer read
    w2_issue(0);
    // intermediate -> LDS: inter op, cast, zero outside the first convolution's output (that is the
    // second one's padding); 4 consecutive channels per register quad
#pragma unroll
    for (int c = 0; c < C1T; ++c)
#pragma unroll
      for (int j = 0; j < PXW; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            v[e] = valid[j] ? acc[c][j][4 * q + e] : 0.f;
            if (p.relu_mid) v[e] = fmaxf(v[e], 0.f);
          }
          const typename Elem<T>::v2 a0 = cvt2<T>(v[0], v[1]), a1 = cvt2<T>(v[2], v[3]);
          const V4 w = {a0[0], a0[1], a1[0], a1[1]};
          *reinterpret_cast<V4*>(Ms + (32 * (PXW * wave + j) + ln) * MS + 32 * c + 8 * q + 4 * g) = w;
        }
    // output pixel slots of this lane
    int moff[PX2];
    bool valid2[PX2];
    long long opix2[PX2];
    const int op0 = th * p.TH2, oq0 = tw * p.TW2;
#pragma unroll
    for (int j = 0; j < PX2; ++j) {
      const int slot = 32 * (PX2 * wave + j) + ln;
      const int oh = slot / p.TW2, ow = slot % p.TW2;
      valid2[j] = oh < p.TH2 && op0 + oh < p.P2 && oq0 + ow < p.Q2;
      const int ohc = valid2[j] ? oh : 0, owc = valid2[j] ? ow : 0;
      moff[j] = (ohc * p.TW + owc) * p.stride2 * MS + 8 * g;
      opix2[j] = (long long)(op0 + ohc) * p.Q2 + oq0 + owc;
    }
    const long long plane2 = (long long)p.P2 * p.Q2;
    f32x16 o[2][PX2];
    // WIDE: operands swapped, pixel-major result o[t][j][r] = out[pixel 8(r/4) + 4g + r%4][c2 = 32t + ln]
    auto run_stages = [&](auto wide_tag) __attribute__((always_inline)) {
      constexpr bool WIDE = decltype(wide_tag)::value;
      for (int stage = 0; stage < nstage; ++stage) {
        const int r = stage % p.R2, sc = stage / p.R2;
        const int c2b = sc / nch2, ch = sc % nch2;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        wg_sync();  // this stage's rows have landed; everyone is done with the previous ones
        if (stage + 1 < nstage) w2_issue(stage + 1);
        if (ch == 0 && r == 0) {
#pragma unroll
          for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j = 0; j < PX2; ++j)
#pragma unroll
              for (int q = 0; q < 16; ++q) o[t][j][q] = 0.f;
        }
        const T* wbuf = reinterpret_cast<const T*>(reinterpret_cast<const char*>(W2b) + (stage & 1) * w2_buf);
        for (int s2 = 0; s2 < p.S2; ++s2) {
          const int tap = (r * p.TW + s2) * MS + 32 * ch;
          const T* wrow = wbuf + (s2 * 64 + ln) * 40 + 8 * g;
          V8 mf[2][PX2], wf[2][2];
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) {
#pragma unroll
            for (int j = 0; j < PX2; ++j) mf[kk][j] = *reinterpret_cast<const V8*>(Ms + moff[j] + tap + 16 * kk);
#pragma unroll
            for (int t = 0; t < 2; ++t) wf[kk][t] = *reinterpret_cast<const V8*>(wrow + 32 * t * 40 + 16 * kk);
          }
#pragma unroll
          for (int kk = 0; kk < 2; ++kk)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
              for (int j = 0; j < PX2; ++j)
                o[t][j] = WIDE ? Elem<T>::mfma32(mf[kk][j], wf[kk][t], o[t][j]) : Elem<T>::mfma32(wf[kk][t], mf[kk][j], o[t][j]);
        }
        if (ch == nch2 - 1 && r == p.R2 - 1) {
          if constexpr (WIDE) {
            // four consecutive pixels of one channel per register quad -> 8-byte LDS writes into this
            // wave's corner, then 16-byte stores (8 pixels of one output row)
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
              for (int j = 0; j < PX2; ++j) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                  float v[4];
#pragma unroll
                  for (int e = 0; e < 4; ++e) {
                    v[e] = o[t][j][4 * q + e];
                    if (p.relu_out) v[e] = fmaxf(v[e], 0.f);
                  }
                  const typename Elem<T>::v2 a0 = cvt2<T>(v[0], v[1]), a1 = cvt2<T>(v[2], v[3]);
                  *reinterpret_cast<V4*>(Ow + ln * kConv2Oss + 8 * q + 4 * g) = V4{a0[0], a0[1], a1[0], a1[1]};
                }
#pragma unroll
                for (int v0 = 0; v0 < 128; v0 += 64) {
                  const int v = v0 + lane;
                  const int chn = v >> 2, sv = v & 3;
                  const int c2 = 64 * c2b + 32 * t + chn;
                  const int slot = 32 * (PX2 * wave + j) + 8 * sv;
                  const int oh = slot / p.TW2, ow = slot - oh * p.TW2;
                  const V8 px = *reinterpret_cast<const V8*>(Ow + chn * kConv2Oss + 8 * sv);
                  if (c2 < p.C2 && oh < p.TH2 && op0 + oh < p.P2 && oq0 + ow < p.Q2)
                    *reinterpret_cast<V8*>(reinterpret_cast<T*>(p.y) + ((long long)n * p.C2 + c2) * plane2 +
                                           (long long)(op0 + oh) * p.Q2 + oq0 + ow) = px;
                }
              }
          } else {
            // o[t][j][q] = out^T[c2 = 64 c2b + 32t + 8(q/4) + 4g + q%4][pixel of lane]
#pragma unroll
            for (int t = 0; t < 2; ++t)
#pragma unroll
              for (int j = 0; j < PX2; ++j) {
                if (!valid2[j]) continue;
#pragma unroll
                for (int q = 0; q < 16; ++q) {
                  const int c2 = 64 * c2b + 32 * t + 8 * (q >> 2) + 4 * g + (q & 3);
                  if (c2 >= p.C2) continue;
                  float v = o[t][j][q];
                  if (p.relu_out) v = fmaxf(v, 0.f);
                  const long long off = ((long long)n * p.C2 + c2) * plane2 + opix2[j];
                  if (p.out_f32)
                    reinterpret_cast<float*>(p.y)[off] = v;
                  else
                    reinterpret_cast<T*>(p.y)[off] = (T)v;
                }
              }
          }
        }
      }
    };
    if (p.wide2) run_stages(std::true_type());
    else run_stages(std::false_type());
    return;
  }

  // ---- second convolution (1x1): W2 blocks go through the LDS the first convolution has finished
  // with.  Inter op on the accumulators, cast: mid^T tile (c, j) regs 8(u%2)..+7 are the
  // B operand of k step u (channels 16u + 4g + {0..3} and 16u + 8 + 4g + {0..3})
  V8 pf[2 * C1T][PXW];
#pragma unroll
  for (int c = 0; c < C1T; ++c)
#pragma unroll
    for (int j = 0; j < PXW; ++j)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[e] = acc[c][j][8 * hh + e];
          if (p.relu_mid) v[e] = fmaxf(v[e], 0.f);
        }
        typename Elem<T>::v2 a0 = cvt2<T>(v[0], v[1]), a1 = cvt2<T>(v[2], v[3]);
        typename Elem<T>::v2 a2 = cvt2<T>(v[4], v[5]), a3 = cvt2<T>(v[6], v[7]);
        V8 w = {a0[0], a0[1], a1[0], a1[1], a2[0], a2[1], a3[0], a3[1]};
        pf[2 * c + hh][j] = w;
      }

  for (int cb = 0; cb < p.C2; cb += c2blk) {
    wg_sync();  // the LDS region is free (first convolution / previous block done)
    if (w2_prefetch && cb == 0) {
#pragma unroll
      for (int k = 0; k < 8; ++k) w2_store(tid + 256 * k, xr[k]);
    } else {
      for (int e = tid; e < c2blk * VPR; e += 256) w2_store(e, w2_load(cb, e));
    }
    wg_sync();
    for (int ct = 0; ct * 32 < c2blk && cb + ct * 32 < p.C2; ++ct) {
      const T* wr = W2s + (32 * ct + ln) * W2S + 4 * g;  // A operand row of this lane
      f32x16 o[PXW];
#pragma unroll
      for (int j = 0; j < PXW; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[j][r] = 0.f;
      V8 wf[2 * C1T];
#pragma unroll
      for (int u = 0; u < 2 * C1T; ++u) {
        const V4 lo = *reinterpret_cast<const V4*>(wr + 16 * u);
        const V4 hi = *reinterpret_cast<const V4*>(wr + 16 * u + 8);
        wf[u] = concat4<V4, V8>(lo, hi);
      }
      if (wide) {
#pragma unroll
        for (int u = 0; u < 2 * C1T; ++u)
#pragma unroll
          for (int j = 0; j < PXW; ++j) o[j] = Elem<T>::mfma32(pf[u][j], wf[u], o[j]);
        // operands swapped: o[j][r] = out[pixel 32j + 8(r/4) + 4g + r%4][c2 = cb + 32ct + ln], four
        // consecutive pixels of one channel per register quad -> one 8-byte LDS write
#pragma unroll
        for (int j = 0; j < PXW; ++j)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              v[e] = o[j][4 * q + e];
              if (p.relu_out) v[e] = fmaxf(v[e], 0.f);
            }
            const typename Elem<T>::v2 a0 = cvt2<T>(v[0], v[1]), a1 = cvt2<T>(v[2], v[3]);
            const V4 w = {a0[0], a0[1], a1[0], a1[1]};
            *reinterpret_cast<V4*>(Os + ln * OSS + 32 * j + 8 * q + 4 * g) = w;
          }
        // 32 rows x SLW/8 vectors of 8 pixels, 64 per pass
#pragma unroll
        for (int v0 = 0; v0 < 32 * (SLW / 8); v0 += 64) {
          const int v = v0 + lane;
          const int ch = v / (SLW / 8), sv = v % (SLW / 8);
          const int c2 = cb + 32 * ct + ch;
          const int slot = SLW * wave + 8 * sv;
          const V8 px = *reinterpret_cast<const V8*>(Os + ch * OSS + 8 * sv);
          if (c2 < p.C2 && slot < nvalid) {
            // write-through (the output streams to memory while the kernel computes: 25.1 -> 23.4 us on the
            // 32 x 64 x 56 x 56 -> 64 -> 256 shape); images past the 32-bit buffer offset keep the streaming store
            if (y_small) {
              const __amdgpu_buffer_rsrc_t yr = __builtin_amdgcn_make_buffer_rsrc(
                  reinterpret_cast<T*>(p.y) + (long long)n * p.C2 * plane, 0, 0x7fffffff, 0x00020000);
              __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, px), yr,
                                                     (unsigned)(((long long)c2 * plane + p0 * p.Q + slot) * 2), 0, kStoreWriteThrough);
            } else {
              __builtin_nontemporal_store(px, reinterpret_cast<V8*>(reinterpret_cast<T*>(p.y) + ((long long)n * p.C2 + c2) * plane + p0 * p.Q + slot));
            }
          }
        }
      } else {
#pragma unroll
        for (int u = 0; u < 2 * C1T; ++u)
#pragma unroll
          for (int j = 0; j < PXW; ++j) o[j] = Elem<T>::mfma32(wf[u], pf[u][j], o[j]);
        // o[j][r] = out^T[c2 = cb + 32ct + 8(r/4) + 4g + r%4][pixel of lane]: for one r the 32 lanes
        // of a half-wave write consecutive pixels of one channel plane
#pragma unroll
        for (int j = 0; j < PXW; ++j) {
          if (!valid[j]) continue;
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int c2 = cb + 32 * ct + 8 * (r >> 2) + 4 * g + (r & 3);
            if (c2 >= p.C2) continue;
            float v = o[j][r];
            if (p.relu_out) v = fmaxf(v, 0.f);
            const long long off = ((long long)n * p.C2 + c2) * plane + opix[j];
            if (p.out_f32)
              reinterpret_cast<float*>(p.y)[off] = v;
            else
              reinterpret_cast<T*>(p.y)[off] = (T)v;
          }
        }
      }
    }
  }
#else
  (void)p;
#endif
}

template <typename T, int C1T, int PXW, int CH, int PX2 = 0>
hipError_t launch_conv_chain(const ConvChainArgs& args, hipStream_t stream) {
  int lds = conv_chain_lds_bytes(args.rows_in, args.cols_in, args.R * args.S, 32 * C1T, CH);
  if (PX2 > 0) {
    const int lds2 = conv_chain2_lds_bytes(128 * PXW, 32 * C1T, args.S2, args.wide2 != 0);
    if (lds2 > lds) lds = lds2;
  }
  auto kern = conv_chain_kernel<T, C1T, PXW, CH, PX2>;
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                            160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  const unsigned grid = (unsigned)args.N * (unsigned)args.tiles_h * (unsigned)args.tiles_w;
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, stream, args);
  return hipGetLastError();
}

// repack W1 into `out` (conv_w1_chunk_bytes * chunks bytes) on `stream`
template <typename T>
hipError_t launch_pack_conv_w1(const ConvChainArgs& args, int C1p, int ch, void* out, hipStream_t stream) {
  const int RS = args.R * args.S;
  const int nchunks = (args.C0 + ch - 1) / ch;
  const long long total = (long long)nchunks * RS * C1p * conv_ch_stride(ch);
  const unsigned grid = (unsigned)((total + 255) / 256);
  hipLaunchKernelGGL(pack_conv_w1_kernel<T>, dim3(grid), dim3(256), 0, stream, reinterpret_cast<const T*>(args.w1),
                     reinterpret_cast<T*>(out), args.C0, args.C1, RS, C1p, ch, total);
  return hipGetLastError();
}

// repack W1 (as launch_pack_conv_w1) and, for a second convolution larger than 1x1, W2
// (conv_w2_chunk_bytes * blocks * chunks bytes) in ONE launch: the first blocks do W1, the rest W2
template <typename T>
__global__ void pack_conv_w12_kernel(const T* __restrict__ w1, T* __restrict__ out1, int C0, int C1, int RS, int C1p,
                                     int ch, long long total1, unsigned blocks1, const T* __restrict__ w2,
                                     T* __restrict__ out2, int C2, int RS2, long long total2) {
  if (blockIdx.x < blocks1) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;  // the packed tensors are far below 2^31 elements
    if (i >= total1) return;
    const unsigned chs = conv_ch_stride(ch);
    const int c = (int)(i % chs);
    unsigned q = i / chs;
    const int c1 = (int)(q % (unsigned)C1p);
    q /= (unsigned)C1p;
    const int rs = (int)(q % (unsigned)RS);
    const int chunk = (int)(q / (unsigned)RS);
    const int c0 = chunk * ch + c;
    T v = (T)0.f;
    if (c < ch && c1 < C1 && c0 < C0) v = w1[((long long)c1 * C0 + c0) * RS + rs];
    out1[i] = v;
  } else {
    const unsigned i = (blockIdx.x - blocks1) * blockDim.x + threadIdx.x;
    if (i >= total2) return;
    const int c = (int)(i % 40u);
    unsigned q = i / 40u;
    const int c2l = (int)(q % 64u);
    q /= 64u;
    const int tap = (int)(q % (unsigned)RS2);
    q /= (unsigned)RS2;
    const int chunk = (int)(q % (unsigned)(C1p / 32));
    const int c2b = (int)(q / (unsigned)(C1p / 32));
    const int c1 = chunk * 32 + c, c2 = c2b * 64 + c2l;
    T v = (T)0.f;
    if (c < 32 && c1 < C1 && c2 < C2) v = w2[((long long)c2 * C1 + c1) * RS2 + tap];
    out2[i] = v;
  }
}

template <typename T>
hipError_t launch_pack_conv_w12(const ConvChainArgs& args, int C1p, int ch, void* out1, void* out2, hipStream_t stream) {
  const int RS = args.R * args.S, RS2 = args.R2 * args.S2;
  const int nchunks = (args.C0 + ch - 1) / ch;
  const long long total1 = (long long)nchunks * RS * C1p * conv_ch_stride(ch);
  const long long total2 = (long long)((args.C2 + 63) / 64) * (C1p / 32) * RS2 * 64 * 40;
  const unsigned blocks1 = (unsigned)((total1 + 255) / 256), blocks2 = (unsigned)((total2 + 255) / 256);
  hipLaunchKernelGGL(pack_conv_w12_kernel<T>, dim3(blocks1 + blocks2), dim3(256), 0, stream,
                     reinterpret_cast<const T*>(args.w1), reinterpret_cast<T*>(out1), args.C0, args.C1, RS, C1p, ch,
                     total1, blocks1, reinterpret_cast<const T*>(args.w2), reinterpret_cast<T*>(out2), args.C2, RS2,
                     total2);
  return hipGetLastError();
}

}  // namespace ditto
