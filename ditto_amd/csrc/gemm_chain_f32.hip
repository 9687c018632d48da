// fp32 / fp64 GEMM -> cast|relu|softmax -> GEMM chain  F = inter(A.B).C  for the reference's fp32, CPU-sized
// configurations (python_test/auto_tensorize/test_hyper_fusion.py:16-21: 512x64 . 64x64 . 64x64; the fp32
// BMM -> softmax -> BMM of benchmark/chimera/cpu/bmm_softmax_bmm.py:64-170).
//
// That configuration is plumbing, not a hot path (0.5 MFLOP per row block), so this kernel is
// plain fp32 FMAs over LDS tiles: a workgroup owns 32 rows of A for one batch entry, walks L in
// tiles of 64, keeps the 32x64 intermediate tile in LDS and its 32xN slice of F in registers.
// (fp64, the reference's ("80", "float64", "float64") row of benchmark/chimera/cuda/bmm_bmm_cuda.py:273-288: the
// same kernel on doubles with tiles of 32 along L, so that K, N up to 128 still fit LDS.)
// Sums run over k, then l, in ascending order in the element type.  Softmax is the online form over the tiles of L: the eight
// threads of a row share its running maximum (exchanged by lane shuffles), each keeps the sum of its own
// probabilities, and the row's slice of F is rescaled when the maximum rises.
#include "gemm_chain_f32.h"

namespace ditto {

namespace {
constexpr int kBM = 32, kMaxD = 128;
template <typename F>
constexpr int tile_l() { return sizeof(F) == 8 ? 32 : 64; }  // intermediate columns per step

__device__ inline float fp_exp2(float x) { return exp2f(x); }
__device__ inline double fp_exp2(double x) { return exp2(x); }
__device__ inline float fp_max(float a, float b) { return fmaxf(a, b); }
__device__ inline double fp_max(double a, double b) { return fmax(a, b); }
__device__ inline float fp_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ inline double fp_fma(double a, double b, double c) { return __builtin_fma(a, b, c); }
}

template <typename F>
__host__ __device__ inline int fp_chain_lds_bytes(int K, int N) {
  constexpr int kBL = tile_l<F>();
  return (kBM * (K + 1) + K * (kBL + 1) + kBL * (N + 1) + kBM * (kBL + 1)) * (int)sizeof(F);
}

template <typename F>
__global__ __launch_bounds__(256) void gemm_chain_fp_kernel(F32ChainArgs p) {
  constexpr int kBL = tile_l<F>();
  extern __shared__ __attribute__((aligned(16))) char smem_fp[];
  const int K = p.K, N = p.N, L = p.L, M = p.M;
  F* As = reinterpret_cast<F*>(smem_fp);  // [32][K+1]
  F* Bs = As + kBM * (K + 1);             // [K][kBL+1]
  F* Cs = Bs + K * (kBL + 1);             // [kBL][N+1]
  F* Ms = Cs + kBL * (N + 1);             // [32][kBL+1]
  const int tid = threadIdx.x;
  const int mb = blockIdx.x % p.mblocks, bz = blockIdx.x / p.mblocks;
  const int m0 = mb * kBM;
  const F* Ag = static_cast<const F*>(p.a) + (long long)bz * p.a_bs;
  const F* Bg = static_cast<const F*>(p.b) + (long long)bz * p.b_bs;
  const F* Cg = static_cast<const F*>(p.c) + (long long)bz * p.c_bs;
  F* Fg = static_cast<F*>(p.f) + (long long)bz * p.f_bs;
  const F zero = 0;

  for (int e = tid; e < kBM * K; e += 256) {
    const int r = e / K, k = e % K;
    As[r * (K + 1) + k] = m0 + r < M ? Ag[(long long)(m0 + r) * p.a_rs + k] : zero;
  }
  const int r = tid >> 3, c8 = tid & 7;  // this thread's row and its column phase
  F acc[kMaxD / 8];
#pragma unroll
  for (int i = 0; i < kMaxD / 8; ++i) acc[i] = zero;

  F mrow = -INFINITY, lsum = zero;  // softmax: running maximum (exp2 domain), this thread's share of the row sum
  const F c2 = (F)p.softmax_scale * (F)1.4426950408889634;

  for (int l0 = 0; l0 < L; l0 += kBL) {
    __syncthreads();
    for (int e = tid; e < K * kBL; e += 256) {
      // consecutive threads read along the contiguous axis of B
      const int k = p.b_lk ? e % K : e / kBL, l = p.b_lk ? e / K : e % kBL;
      F v = zero;
      if (l0 + l < L) v = p.b_lk ? Bg[(long long)(l0 + l) * p.b_rs + k] : Bg[(long long)k * p.b_rs + l0 + l];
      Bs[k * (kBL + 1) + l] = v;
    }
    for (int e = tid; e < kBL * N; e += 256) {
      const int l = e / N, n = e % N;
      Cs[l * (N + 1) + n] = l0 + l < L ? Cg[(long long)(l0 + l) * p.c_rs + n] : zero;
    }
    __syncthreads();
    F sv[kBL / 8];
#pragma unroll
    for (int j = 0; j < kBL / 8; ++j) {
      const int l = c8 + 8 * j;
      F s = zero;
      for (int k = 0; k < K; ++k) s = fp_fma(As[r * (K + 1) + k], Bs[k * (kBL + 1) + l], s);
      if (p.relu) s = fp_max(s, zero);
      sv[j] = s;
    }
    if (p.softmax) {
      F mx = -INFINITY;
#pragma unroll
      for (int j = 0; j < kBL / 8; ++j) {
        sv[j] = l0 + c8 + 8 * j < L ? sv[j] * c2 : (F)-INFINITY;  // keys past L take no part
        mx = fp_max(mx, sv[j]);
      }
      // the row's eight threads are eight consecutive lanes
      mx = fp_max(mx, __shfl_xor(mx, 1));
      mx = fp_max(mx, __shfl_xor(mx, 2));
      mx = fp_max(mx, __shfl_xor(mx, 4));
      const F mnew = fp_max(mrow, mx);  // finite: every tile holds at least one key
      const F alpha = fp_exp2(mrow - mnew);
      mrow = mnew;
      lsum *= alpha;
#pragma unroll
      for (int i = 0; i < kMaxD / 8; ++i) acc[i] *= alpha;
#pragma unroll
      for (int j = 0; j < kBL / 8; ++j) {
        sv[j] = fp_exp2(sv[j] - mnew);
        lsum += sv[j];
      }
    }
#pragma unroll
    for (int j = 0; j < kBL / 8; ++j) Ms[r * (kBL + 1) + c8 + 8 * j] = sv[j];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kMaxD / 8; ++i) {
      const int n = c8 + 8 * i;
      if (n < N) {
        F s = acc[i];
        for (int l = 0; l < kBL; ++l) s = fp_fma(Ms[r * (kBL + 1) + l], Cs[l * (N + 1) + n], s);
        acc[i] = s;
      }
    }
  }
  F inv = 1;
  if (p.softmax) {
    lsum += __shfl_xor(lsum, 1);
    lsum += __shfl_xor(lsum, 2);
    lsum += __shfl_xor(lsum, 4);
    inv = (F)1 / lsum;
  }
  if (m0 + r < M) {
#pragma unroll
    for (int i = 0; i < kMaxD / 8; ++i) {
      const int n = c8 + 8 * i;
      if (n < N) Fg[(long long)(m0 + r) * p.f_rs + n] = p.relu_out ? fp_max(acc[i] * inv, zero) : acc[i] * inv;
    }
  }
}

int f32_chain_lds_bytes_host(int K, int N, int f64) { return f64 ? fp_chain_lds_bytes<double>(K, N) : fp_chain_lds_bytes<float>(K, N); }
int f32_chain_max_dim() { return kMaxD; }

template <typename F>
static hipError_t launch_fp(const F32ChainArgs& args, hipStream_t stream) {
  const int lds = fp_chain_lds_bytes<F>(args.K, args.N);
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_chain_fp_kernel<F>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  const unsigned grid = (unsigned)args.mblocks * (unsigned)args.batch;
  hipLaunchKernelGGL(gemm_chain_fp_kernel<F>, dim3(grid), dim3(256), lds, stream, args);
  return hipGetLastError();
}

hipError_t launch_gemm_chain_f32(const F32ChainArgs& args, hipStream_t stream) {
  return args.f64 ? launch_fp<double>(args, stream) : launch_fp<float>(args, stream);
}

}  // namespace ditto
