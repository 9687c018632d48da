// fp32 GEMM -> cast|relu|softmax -> GEMM chain  F = inter(A.B).C  for the reference's fp32, CPU-sized
// configurations (python_test/auto_tensorize/test_hyper_fusion.py:16-21: 512x64 . 64x64 . 64x64; the fp32
// BMM -> softmax -> BMM of benchmark/chimera/cpu/bmm_softmax_bmm.py:64-170).
//
// That configuration is plumbing, not a hot path (0.5 MFLOP per row block), so this kernel is
// plain fp32 FMAs over LDS tiles: a workgroup owns 32 rows of A for one batch entry, walks L in
// tiles of 64, keeps the 32x64 intermediate tile in LDS and its 32xN slice of F in registers.
// Sums run over k, then l, in ascending order in fp32.  Softmax is the online form over the tiles of L: the eight
// threads of a row share its running maximum (exchanged by lane shuffles), each keeps the sum of its own
// probabilities, and the row's slice of F is rescaled when the maximum rises.
#include "gemm_chain_f32.h"

namespace ditto {

namespace {
constexpr int kBM = 32, kBL = 64, kMaxD = 128;
}

__host__ __device__ inline int f32_chain_lds_bytes(int K, int N) {
  return (kBM * (K + 1) + K * (kBL + 1) + kBL * (N + 1) + kBM * (kBL + 1)) * 4;
}

__global__ __launch_bounds__(256) void gemm_chain_f32_kernel(F32ChainArgs p) {
  extern __shared__ float smem_f32[];
  const int K = p.K, N = p.N, L = p.L, M = p.M;
  float* As = smem_f32;                   // [32][K+1]
  float* Bs = As + kBM * (K + 1);         // [K][65]
  float* Cs = Bs + K * (kBL + 1);         // [64][N+1]
  float* Ms = Cs + kBL * (N + 1);         // [32][65]
  const int tid = threadIdx.x;
  const int mb = blockIdx.x % p.mblocks, bz = blockIdx.x / p.mblocks;
  const int m0 = mb * kBM;
  const float* Ag = p.a + (long long)bz * p.a_bs;
  const float* Bg = p.b + (long long)bz * p.b_bs;
  const float* Cg = p.c + (long long)bz * p.c_bs;
  float* Fg = p.f + (long long)bz * p.f_bs;

  for (int e = tid; e < kBM * K; e += 256) {
    const int r = e / K, k = e % K;
    As[r * (K + 1) + k] = m0 + r < M ? Ag[(long long)(m0 + r) * p.a_rs + k] : 0.f;
  }
  const int r = tid >> 3, c8 = tid & 7;  // this thread's row and its column phase
  float acc[kMaxD / 8];
#pragma unroll
  for (int i = 0; i < kMaxD / 8; ++i) acc[i] = 0.f;

  float mrow = -INFINITY, lsum = 0.f;  // softmax: running maximum (exp2 domain), this thread's share of the row sum
  const float c2 = p.scale_log2;

  for (int l0 = 0; l0 < L; l0 += kBL) {
    __syncthreads();
    for (int e = tid; e < K * kBL; e += 256) {
      // consecutive threads read along the contiguous axis of B
      const int k = p.b_lk ? e % K : e / kBL, l = p.b_lk ? e / K : e % kBL;
      float v = 0.f;
      if (l0 + l < L) v = p.b_lk ? Bg[(long long)(l0 + l) * p.b_rs + k] : Bg[(long long)k * p.b_rs + l0 + l];
      Bs[k * (kBL + 1) + l] = v;
    }
    for (int e = tid; e < kBL * N; e += 256) {
      const int l = e / N, n = e % N;
      Cs[l * (N + 1) + n] = l0 + l < L ? Cg[(long long)(l0 + l) * p.c_rs + n] : 0.f;
    }
    __syncthreads();
    float sv[kBL / 8];
#pragma unroll
    for (int j = 0; j < kBL / 8; ++j) {
      const int l = c8 + 8 * j;
      float s = 0.f;
      for (int k = 0; k < K; ++k) s = __builtin_fmaf(As[r * (K + 1) + k], Bs[k * (kBL + 1) + l], s);
      if (p.relu) s = fmaxf(s, 0.f);
      sv[j] = s;
    }
    if (p.softmax) {
      float mx = -INFINITY;
#pragma unroll
      for (int j = 0; j < kBL / 8; ++j) {
        sv[j] = l0 + c8 + 8 * j < L ? sv[j] * c2 : -INFINITY;  // keys past L take no part
        mx = fmaxf(mx, sv[j]);
      }
      // the row's eight threads are eight consecutive lanes
      mx = fmaxf(mx, __shfl_xor(mx, 1));
      mx = fmaxf(mx, __shfl_xor(mx, 2));
      mx = fmaxf(mx, __shfl_xor(mx, 4));
      const float mnew = fmaxf(mrow, mx);  // finite: every tile holds at least one key
      const float alpha = exp2f(mrow - mnew);
      mrow = mnew;
      lsum *= alpha;
#pragma unroll
      for (int i = 0; i < kMaxD / 8; ++i) acc[i] *= alpha;
#pragma unroll
      for (int j = 0; j < kBL / 8; ++j) {
        sv[j] = exp2f(sv[j] - mnew);
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
        float s = acc[i];
        for (int l = 0; l < kBL; ++l) s = __builtin_fmaf(Ms[r * (kBL + 1) + l], Cs[l * (N + 1) + n], s);
        acc[i] = s;
      }
    }
  }
  float inv = 1.f;
  if (p.softmax) {
    lsum += __shfl_xor(lsum, 1);
    lsum += __shfl_xor(lsum, 2);
    lsum += __shfl_xor(lsum, 4);
    inv = 1.f / lsum;
  }
  if (m0 + r < M) {
#pragma unroll
    for (int i = 0; i < kMaxD / 8; ++i) {
      const int n = c8 + 8 * i;
      if (n < N) Fg[(long long)(m0 + r) * p.f_rs + n] = p.relu_out ? fmaxf(acc[i] * inv, 0.f) : acc[i] * inv;
    }
  }
}

int f32_chain_lds_bytes_host(int K, int N) { return f32_chain_lds_bytes(K, N); }
int f32_chain_max_dim() { return kMaxD; }

hipError_t launch_gemm_chain_f32(const F32ChainArgs& args, hipStream_t stream) {
  const int lds = f32_chain_lds_bytes(args.K, args.N);
  static thread_local int configured_dev = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_chain_f32_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
  }
  const unsigned grid = (unsigned)args.mblocks * (unsigned)args.batch;
  hipLaunchKernelGGL(gemm_chain_f32_kernel, dim3(grid), dim3(256), lds, stream, args);
  return hipGetLastError();
}

}  // namespace ditto
