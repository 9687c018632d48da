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
// Work split: a workgroup of 4 waves owns 128*QT rows of A for one batch entry; each
// wave owns 32*QT rows and keeps their A fragments in VGPRs for the whole kernel.
// The L axis is walked in steps of 64: B and C tiles are staged through LDS (double
// buffered, one barrier per step) and shared by the 4 waves.
#pragma once
#include "common.h"

namespace ditto {

struct BmmChainArgs {
  const void* a;
  const void* b;
  const void* c;
  void* f;
  long long a_bs, b_bs, c_bs, f_bs;  // batch strides, elements
  int a_rs, b_rs, c_rs, f_rs;        // row strides, elements
  int M, N, K, L, batch;
  int mblocks;       // workgroups per batch entry
  float scale_log2;  // softmax: scale * log2(e)
  int relu;          // inter = relu instead of cast (non-softmax kernels)
  int out_f32;       // write F as fp32 instead of T
};

constexpr int kInterCast = 0;
constexpr int kInterSoftmax = 2;

constexpr int kBN = 64;  // L step
constexpr float kLazy = 8.0f;  // log2 of the slack allowed before the running maximum is raised
constexpr int kNW = 4;   // waves per workgroup

// Row stride (elements) of a row-major 16-bit LDS tile that is read with transpose
// reads: 4 consecutive rows x 64 B must fall into different banks, which holds when
// the stride in bytes is 64 mod 128.
__host__ __device__ constexpr int tr_stride(int cols) { return (cols % 64 == 32) ? cols : cols + 32; }
// Row stride of a tile read with plain 16-byte row reads (one row per lane).
__host__ __device__ constexpr int row_stride(int cols) { return cols + 8; }

template <int D, bool B_KL>
__host__ __device__ constexpr int bmm_chain_lds_bytes() {
  const int btile = B_KL ? D * tr_stride(kBN) : kBN * row_stride(D);
  const int ctile = kBN * tr_stride(D);
  return 2 * (btile + ctile) * 2;
}

template <typename T, int D, int QT, int INTER, bool B_KL>
__global__ __launch_bounds__(256) void bmm_chain_kernel(BmmChainArgs p) {
  typedef typename Elem<T>::v8 V8;
  typedef typename Elem<T>::v4 V4;
  constexpr int BM = kNW * 32 * QT;
  constexpr int BSTR = B_KL ? tr_stride(kBN) : row_stride(D);
  constexpr int BTILE = B_KL ? D * BSTR : kBN * BSTR;
  constexpr int CSTR = tr_stride(D);
  constexpr int CTILE = kBN * CSTR;
  constexpr int NCH = kBN * D / 8 / 256;  // 16-byte chunks per thread per tile
  static_assert(NCH >= 1 && (kBN * D / 8) % 256 == 0, "tile must split evenly over 256 threads");

  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  T* const Bs = reinterpret_cast<T*>(smem_raw);  // [2][BTILE]
  T* const Cs = Bs + 2 * BTILE;                  // [2][CTILE]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, g = lane >> 5;
  const int i16 = lane & 15, h = (lane >> 4) & 1;

  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
  const int mb = lid % p.mblocks;
  const int bz = lid / p.mblocks;
  const T* __restrict__ Ag = reinterpret_cast<const T*>(p.a) + (long long)bz * p.a_bs;
  const T* __restrict__ Bg = reinterpret_cast<const T*>(p.b) + (long long)bz * p.b_bs;
  const T* __restrict__ Cg = reinterpret_cast<const T*>(p.c) + (long long)bz * p.c_bs;
  const int m_wave = mb * BM + wave * 32 * QT;
  const int M = p.M, N = p.N, K = p.K, L = p.L;

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

  // ---- global -> register staging of one (B, C) tile pair
  V8 breg[NCH], creg[NCH];
  auto load_tiles = [&](int l0) {
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int ch = tid + 256 * c;
      V8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (B_KL) {
        const int k = ch / (kBN / 8), l = l0 + (ch % (kBN / 8)) * 8;
        if (k < K && l < L) v = *reinterpret_cast<const V8*>(Bg + (long long)k * p.b_rs + l);
      } else {
        const int l = l0 + ch / (D / 8), k = (ch % (D / 8)) * 8;
        if (l < L && k < K) v = *reinterpret_cast<const V8*>(Bg + (long long)l * p.b_rs + k);
      }
      breg[c] = v;
      V8 w = {0, 0, 0, 0, 0, 0, 0, 0};
      {
        const int l = l0 + ch / (D / 8), n = (ch % (D / 8)) * 8;
        if (l < L && n < N) w = *reinterpret_cast<const V8*>(Cg + (long long)l * p.c_rs + n);
      }
      creg[c] = w;
    }
  };
  auto store_tiles = [&](int buf) {
    T* bs = Bs + buf * BTILE;
    T* cs = Cs + buf * CTILE;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const int ch = tid + 256 * c;
      if (B_KL) {
        *reinterpret_cast<V8*>(bs + (ch / (kBN / 8)) * BSTR + (ch % (kBN / 8)) * 8) = breg[c];
      } else {
        *reinterpret_cast<V8*>(bs + (ch / (D / 8)) * BSTR + (ch % (D / 8)) * 8) = breg[c];
      }
      *reinterpret_cast<V8*>(cs + (ch / (D / 8)) * CSTR + (ch % (D / 8)) * 8) = creg[c];
    }
  };

  // ---- accumulators of F^T: o[t][j][r] = F^T[32t + 8(r/4) + 4g + r%4][32j + ln]
  f32x16 o[D / 32][QT];
#pragma unroll
  for (int t = 0; t < D / 32; ++t)
#pragma unroll
    for (int j = 0; j < QT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) o[t][j][r] = 0.f;
  float mrow[QT], lsum[QT];
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    mrow[j] = -INFINITY;
    lsum[j] = 0.f;
  }
  const float c2 = p.scale_log2;

  const int ntiles = (L + kBN - 1) / kBN;
  load_tiles(0);
  store_tiles(0);
  __syncthreads();

  for (int it = 0; it < ntiles; ++it) {
    const int buf = it & 1;
    const int l0 = it * kBN;
    if (it + 1 < ntiles) load_tiles(l0 + kBN);
    const T* bs = Bs + buf * BTILE;
    const T* cs = Cs + buf * CTILE;

    // ---- first contraction, transposed: s[i][j] = (B^T tile i) . (A^T tile j)
    f32x16 s[2][QT];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < QT; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) s[i][j][r] = 0.f;
#pragma unroll
    for (int st = 0; st < D / 16; ++st) {
      V8 bf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        if (B_KL) {
          // rows of the LDS tile are k, columns are l: transpose read
          const T* q = bs + (16 * st + 8 * g + (i16 >> 2)) * BSTR + 32 * i + 16 * h + 4 * (i16 & 3);
          V4 lo = lds_read_tr4<T>(q);
          V4 hi = lds_read_tr4<T>(q + 4 * BSTR);
          bf[i] = concat4<V4, V8>(lo, hi);
        } else {
          bf[i] = *reinterpret_cast<const V8*>(bs + (32 * i + ln) * BSTR + 16 * st + 8 * g);
        }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < QT; ++j) s[i][j] = Elem<T>::mfma32(bf[i], af[j][st], s[i][j]);
    }

    // ---- inter-path op on the accumulator registers
    if (INTER == kInterSoftmax) {
      if (l0 + kBN > L) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int l = l0 + 32 * i + 8 * (r >> 2) + 4 * g + (r & 3);
            if (l >= L) {
#pragma unroll
              for (int j = 0; j < QT; ++j) s[i][j][r] = -INFINITY;
            }
          }
      }
#pragma unroll
      for (int j = 0; j < QT; ++j) {
        float mx = s[0][j][0];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[i][j][r]);
        mx = pair_max(mx) * c2;
        // Lazy rescale: the running maximum only has to bound the scores well enough that
        // exp2 cannot overflow, so it is raised (and the accumulators rescaled) only when
        // some row of the wave exceeds it by more than 2^kLazy.  Rows keep a stale maximum
        // otherwise; the final division by the row sum cancels it exactly.
        if (__builtin_amdgcn_ballot_w64(mx > mrow[j] + kLazy) != 0) {
          const float mnew = fmaxf(mrow[j], mx);
          const float alpha = __builtin_amdgcn_exp2f(mrow[j] - mnew);
          mrow[j] = mnew;
          lsum[j] *= alpha;
#pragma unroll
          for (int t = 0; t < D / 32; ++t)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[t][j][r] *= alpha;
        }
        const float mcur = mrow[j];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            s[i][j][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i][j][r], c2, -mcur));
      }
    } else if (p.relu) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < QT; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) s[i][j][r] = fmaxf(s[i][j][r], 0.f);
    }

    // ---- second contraction: o[t][j] += (C^T tile t, l step u) . (P^T tile j, l step u)
    // l step u covers tile rows 16u..16u+15; half-wave g supplies rows
    // 16u + 4g + {0..3} and 16u + 8 + 4g + {0..3} (the accumulator layout of s).
#pragma unroll
    for (int u = 0; u < kBN / 16; ++u) {
      V8 pf[QT];
#pragma unroll
      for (int j = 0; j < QT; ++j) {
        const int i = u >> 1, r0 = 8 * (u & 1);
        typename Elem<T>::v2 p0 = cvt2<T>(s[i][j][r0 + 0], s[i][j][r0 + 1]);
        typename Elem<T>::v2 p1 = cvt2<T>(s[i][j][r0 + 2], s[i][j][r0 + 3]);
        typename Elem<T>::v2 p2 = cvt2<T>(s[i][j][r0 + 4], s[i][j][r0 + 5]);
        typename Elem<T>::v2 p3 = cvt2<T>(s[i][j][r0 + 6], s[i][j][r0 + 7]);
        if (INTER == kInterSoftmax) {
          // the row sum is taken over the ROUNDED probabilities, i.e. exactly the values
          // that enter the second contraction
          lsum[j] = Elem<T>::add_pair(p0, lsum[j]);
          lsum[j] = Elem<T>::add_pair(p1, lsum[j]);
          lsum[j] = Elem<T>::add_pair(p2, lsum[j]);
          lsum[j] = Elem<T>::add_pair(p3, lsum[j]);
        }
        V8 v = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
        pf[j] = v;
      }
#pragma unroll
      for (int t = 0; t < D / 32; ++t) {
        const T* q = cs + (16 * u + 4 * g + (i16 >> 2)) * CSTR + 32 * t + 16 * h + 4 * (i16 & 3);
        V4 lo = lds_read_tr4<T>(q);
        V4 hi = lds_read_tr4<T>(q + 8 * CSTR);
        V8 cf = concat4<V4, V8>(lo, hi);
#pragma unroll
        for (int j = 0; j < QT; ++j) o[t][j] = Elem<T>::mfma32(cf, pf[j], o[t][j]);
      }
    }

    if (it + 1 < ntiles) store_tiles(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: normalise (softmax), cast, store 4 contiguous columns per lane
#pragma unroll
  for (int j = 0; j < QT; ++j) {
    float inv = 1.f;
    if (INTER == kInterSoftmax) inv = 1.f / pair_sum(lsum[j]);
    const int row = m_wave + 32 * j + ln;
    if (row >= M) continue;
#pragma unroll
    for (int t = 0; t < D / 32; ++t)
#pragma unroll
      for (int q4 = 0; q4 < 4; ++q4) {
        const int n = 32 * t + 8 * q4 + 4 * g;
        if (n >= N) continue;
        const float v0 = o[t][j][4 * q4 + 0] * inv, v1 = o[t][j][4 * q4 + 1] * inv;
        const float v2 = o[t][j][4 * q4 + 2] * inv, v3 = o[t][j][4 * q4 + 3] * inv;
        const long long off = (long long)bz * p.f_bs + (long long)row * p.f_rs + n;
        if (p.out_f32) {
          f32x4 w = {v0, v1, v2, v3};
          *reinterpret_cast<f32x4*>(reinterpret_cast<float*>(p.f) + off) = w;
        } else {
          typename Elem<T>::v2 a0 = cvt2<T>(v0, v1), a1 = cvt2<T>(v2, v3);
          V4 w = {a0[0], a0[1], a1[0], a1[1]};
          *reinterpret_cast<V4*>(reinterpret_cast<T*>(p.f) + off) = w;
        }
      }
  }
}

// Host-side launcher for one instantiation.
template <typename T, int D, int QT, int INTER, bool B_KL>
hipError_t launch_bmm_chain(const BmmChainArgs& args, hipStream_t stream) {
  constexpr int lds = bmm_chain_lds_bytes<D, B_KL>();
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
