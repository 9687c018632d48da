// int8 GEMM -> requantise -> GEMM chain on gfx950:  E = sat_i8(rne((A.B) * scale[l])) . D
//
// The reference declares int8 -> int32 for its GEMM chain (benchmark/chimera/cuda/
// bmm_bmm_cuda.py:273-288) and casts the middle result with a wrapping astype("int8")
// (:114-118); the requantise step (per-column scale, round to nearest even, saturate to
// [-128,127]) is this build's workload definition.  All arithmetic is exact integer except
// the requantise, which is one fp32 multiply and one round-to-nearest-even: results are
// bit-identical to the CPU checker.
//
// A workgroup of 4 waves owns 64 rows of A.  Phase 1 computes the middle result TRANSPOSED
// (mid^T = B^T.A^T) with v_mfma_i32_32x32x32_i8 so that each lane ends up with 4 consecutive
// l for one row m, requantises in registers and writes the int8 row block mid[64][L] to LDS
// (it never goes to HBM).  Phase 2 walks N in chunks of 256 and multiplies the LDS-resident
// mid by D.  B and D are row-major with the contraction index as the ROW index, the opposite
// of what an MFMA operand wants (16 consecutive k per lane); they are staged row-major in LDS
// and read with the transposing LDS read ds_read_b64_tr_b8.
#include "common.h"
#include "gemm_chain_i8.h"

namespace ditto {

namespace i8 {
constexpr int BM = 64;     // rows of A per workgroup
constexpr int KC = 64;     // contraction chunk staged per step
constexpr int WC = 256;    // width of a staged weight chunk (columns of B / D)
constexpr int ASTR = 80;   // LDS row stride of the A tile: 64 + 16, conflict-free 16-byte row reads
constexpr int WSTR = 288;  // LDS row stride of a weight tile: 8 rows x 32 B of a transpose read
                           // fall into different banks when the stride is 32 mod 64 bytes
constexpr int MIDPAD = 16;
}  // namespace i8

__host__ __device__ inline int i8_chain_lds_bytes(int Lp) {
  return 2 * i8::BM * i8::ASTR + 2 * i8::KC * i8::WSTR + i8::BM * (Lp + i8::MIDPAD) + Lp * 4;
}

// 8 k-rows x 16 columns of a row-major int8 LDS tile, transposed: lane i of each 16-lane
// group receives column c0+i, rows r0..r0+7 when lane s points at tile[r0 + s/2][c0 + 8*(s%2)].
__device__ __forceinline__ i32x2 lds_read_tr8(const int8_t* p) {
  return __builtin_amdgcn_ds_read_tr8_b64_v2i32((DITTO_LDS i32x2*)p);
}

__device__ __forceinline__ int requant_i8(int acc, float s) {
  float v = __builtin_rintf((float)acc * s);
  v = fminf(fmaxf(v, -128.f), 127.f);
  return (int)v;
}

__global__ __launch_bounds__(256) void gemm_chain_i8_kernel(I8ChainArgs p) {
  using namespace i8;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  int8_t* const As = reinterpret_cast<int8_t*>(smem_raw);  // [2][BM*ASTR]
  int8_t* const Ws = As + 2 * BM * ASTR;                   // [2][KC*WSTR]
  const int MIDSTR = p.Lp + MIDPAD;
  int8_t* const mid = Ws + 2 * KC * WSTR;                  // [BM][MIDSTR]
  float* const sc = reinterpret_cast<float*>(mid + BM * MIDSTR);  // [Lp]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, g = lane >> 5;
  const int i16 = lane & 15, h = (lane >> 4) & 1;
  const unsigned lid = xcd_remap(blockIdx.x, gridDim.x);
  const int mb = lid % p.mblocks, bz = lid / p.mblocks;
  const int m0 = mb * BM;
  const int M = p.M, N = p.N, K = p.K, L = p.L, Lp = p.Lp;
  const int8_t* __restrict__ Ag = p.a + (long long)bz * p.a_bs;
  const int8_t* __restrict__ Bg = p.b + (long long)bz * p.b_bs;
  const int8_t* __restrict__ Dg = p.d + (long long)bz * p.d_bs;
  int32_t* __restrict__ Eg = p.e + (long long)bz * p.e_bs;

  for (int l = tid; l < Lp; l += 256) sc[l] = l < L ? (p.scale ? p.scale[l] : p.scale_uniform) : 0.f;

  // ---- staging helpers (global -> registers -> LDS), 16 bytes per access, zero filled
  i32x4 areg, wreg[4];
  auto load_a = [&](int k0) {
    const int r = tid >> 2, c = (tid & 3) * 16;
    i32x4 v = {0, 0, 0, 0};
    if (m0 + r < M && k0 + c < K) v = *reinterpret_cast<const i32x4*>(Ag + (long long)(m0 + r) * p.a_rs + k0 + c);
    areg = v;
  };
  auto store_a = [&](int buf) {
    const int r = tid >> 2, c = (tid & 3) * 16;
    *reinterpret_cast<i32x4*>(As + buf * BM * ASTR + r * ASTR + c) = areg;
  };
  // weight tile: rows r0..r0+63 (< rmax) and columns c0..c0+255 (< cmax) of W
  auto load_w = [&](const int8_t* __restrict__ W, int rs, int r0, int rmax, int c0, int cmax) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ch = tid + 256 * i;
      const int r = ch >> 4, c = (ch & 15) * 16;
      i32x4 v = {0, 0, 0, 0};
      if (r0 + r < rmax && c0 + c < cmax) v = *reinterpret_cast<const i32x4*>(W + (long long)(r0 + r) * rs + c0 + c);
      wreg[i] = v;
    }
  };
  auto store_w = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int ch = tid + 256 * i;
      const int r = ch >> 4, c = (ch & 15) * 16;
      *reinterpret_cast<i32x4*>(Ws + buf * KC * WSTR + r * WSTR + c) = wreg[i];
    }
  };
  // operand fragment of a weight tile for the 32-wide column tile `ct` of this wave and the
  // 32-deep contraction step `ks`: lane (ln, g) receives W[32ks + 16g + 0..15][64*wave + 32ct + ln]
  auto w_frag = [&](const int8_t* ws, int ks, int ct) -> i32x4 {
    const int8_t* q = ws + (32 * ks + 16 * g + (i16 >> 1)) * WSTR + 64 * wave + 32 * ct + 16 * h + 8 * (i16 & 1);
    const i32x2 lo = lds_read_tr8(q);
    const i32x2 hi = lds_read_tr8(q + 8 * WSTR);
    i32x4 r = {lo[0], lo[1], hi[0], hi[1]};
    return r;
  };

  // ================= phase 1: mid = requant(A.B), kept in LDS =================
  for (int lc = 0; lc < Lp; lc += WC) {
    i32x16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;
    const int nk = (K + KC - 1) / KC;
    __syncthreads();  // previous users of the staging buffers are done
    load_a(0);
    load_w(Bg, p.b_rs, 0, K, lc, L);
    store_a(0);
    store_w(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
      const int buf = kt & 1;
      if (kt + 1 < nk) {
        load_a((kt + 1) * KC);
        load_w(Bg, p.b_rs, (kt + 1) * KC, K, lc, L);
      }
      const int8_t* as = As + buf * BM * ASTR;
      const int8_t* ws = Ws + buf * KC * WSTR;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        i32x4 af[2], bf[2];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
          af[mt] = *reinterpret_cast<const i32x4*>(as + (32 * mt + ln) * ASTR + 32 * ks + 16 * g);
#pragma unroll
        for (int lt = 0; lt < 2; ++lt) bf[lt] = w_frag(ws, ks, lt);
#pragma unroll
        for (int lt = 0; lt < 2; ++lt)
#pragma unroll
          for (int mt = 0; mt < 2; ++mt)
            acc[lt][mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[lt], af[mt], acc[lt][mt], 0, 0, 0);
      }
      if (kt + 1 < nk) {
        store_a(buf ^ 1);
        store_w(buf ^ 1);
      }
      __syncthreads();
    }
    // requantise: acc[lt][mt][r] = mid^T[l][m], l = lc + 64*wave + 32lt + 8(r/4) + 4g + r%4,
    // m = 32mt + ln; 4 consecutive l pack into one dword of mid[m][l..l+3]
#pragma unroll
    for (int lt = 0; lt < 2; ++lt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int l = lc + 64 * wave + 32 * lt + 8 * q + 4 * g;
        const f32x4 s4 = *reinterpret_cast<const f32x4*>(sc + l);
#pragma unroll
        for (int mt = 0; mt < 2; ++mt) {
          const int b0 = requant_i8(acc[lt][mt][4 * q + 0], s4[0]);
          const int b1 = requant_i8(acc[lt][mt][4 * q + 1], s4[1]);
          const int b2 = requant_i8(acc[lt][mt][4 * q + 2], s4[2]);
          const int b3 = requant_i8(acc[lt][mt][4 * q + 3], s4[3]);
          const int packed = (b0 & 0xff) | ((b1 & 0xff) << 8) | ((b2 & 0xff) << 16) | ((unsigned)b3 << 24);
          *reinterpret_cast<int*>(mid + (32 * mt + ln) * MIDSTR + l) = packed;
        }
      }
  }
  __syncthreads();

  // ================= phase 2: E = mid.D, N walked in chunks of 256 =================
  const int nl = Lp / KC;
  for (int nc = 0; nc < N; nc += WC) {
    i32x16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a][b][r] = 0;
    load_w(Dg, p.d_rs, 0, L, nc, N);
    store_w(0);
    __syncthreads();
    for (int lt = 0; lt < nl; ++lt) {
      const int buf = lt & 1;
      if (lt + 1 < nl) load_w(Dg, p.d_rs, (lt + 1) * KC, L, nc, N);
      const int8_t* ws = Ws + buf * KC * WSTR;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        i32x4 af[2], bf[2];
#pragma unroll
        for (int mt = 0; mt < 2; ++mt)
          af[mt] = *reinterpret_cast<const i32x4*>(mid + (32 * mt + ln) * MIDSTR + lt * KC + 32 * ks + 16 * g);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) bf[nt] = w_frag(ws, ks, nt);
#pragma unroll
        for (int nt = 0; nt < 2; ++nt)
#pragma unroll
          for (int mt = 0; mt < 2; ++mt)
            acc[nt][mt] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[mt], bf[nt], acc[nt][mt], 0, 0, 0);
      }
      if (lt + 1 < nl) store_w(buf ^ 1);
      __syncthreads();
    }
    // acc[nt][mt][r] = E[m][n], m = m0 + 32mt + 8(r/4) + 4g + r%4, n = nc + 64*wave + 32nt + ln:
    // the 32 lanes of a half-wave write 128 contiguous bytes of one output row
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int n = nc + 64 * wave + 32 * nt + ln;
      if (n >= N) continue;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + 32 * mt + 8 * (r >> 2) + 4 * g + (r & 3);
          if (m < M) Eg[(long long)m * p.e_rs + n] = acc[nt][mt][r];
        }
    }
  }
}

int i8_chain_lds_bytes_host(int Lp) { return i8_chain_lds_bytes(Lp); }

hipError_t launch_gemm_chain_i8(const I8ChainArgs& args, hipStream_t stream) {
  const int lds = i8_chain_lds_bytes(args.Lp);
  static thread_local int configured_dev = -1;
  static thread_local int configured_lds = 0;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (configured_dev != dev || configured_lds < lds) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_chain_i8_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    configured_dev = dev;
    configured_lds = 160 * 1024;
  }
  const unsigned grid = (unsigned)args.mblocks * (unsigned)args.batch;
  hipLaunchKernelGGL(gemm_chain_i8_kernel, dim3(grid), dim3(256), lds, stream, args);
  return hipGetLastError();
}

}  // namespace ditto
