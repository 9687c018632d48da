// CPU target of the fused two-contraction chain  F = epilogue(inter(A.B).C)  on fp32 / fp64 row-major operands.
//
// What the reference's TensorizeCPU produces for this chain (src/auto_tensorize/hyper_fusion_cpu.cc:853-907,
// 1553-1614): the outer loops of the second contraction are split by the tiling factors of a CPUTensorizeParam and
// run in parallel, the first contraction is computed at the second one's last common loop into a tile that stays
// in cache, and both contractions run on a register-tile micro-kernel reached through call_extern
// ("<prefix>_update" / "<prefix>_reset", python/ditto/auto_tensorize/intrinsic.py:646-674; 6 x 16 fp32 on AVX2,
// :292-416).  Here the nest is written out once, its tiling comes in through the descriptor, and the micro-kernels
// are either the ones below or functions the caller hands in (compiled from the source that cpu_intrin generates).
//
// Built by g++ into libditto_chain_cpu.so, a library of its own: nothing on the HIP path links or loads it.
#include <immintrin.h>
#include <omp.h>
#include <stdint.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <limits>
#include <vector>

#define DITTO_CPU_ABI_VERSION 1

extern "C" {

// `update` micro-kernel:  c[mi][ni] += a[mi][kc] . b[kc][ni]  on row-major tiles with leading dimensions
// lda, ldb, ldc (elements); mi and ni are the intrinsic's own constants.
typedef void (*ditto_cpu_update_f32)(const float* a, long lda, const float* b, long ldb, float* c, long ldc, long kc);
typedef void (*ditto_cpu_update_f64)(const double* a, long lda, const double* b, long ldb, double* c, long ldc, long kc);

typedef struct ditto_cpu_chain_desc {
  int32_t abi_version;  // DITTO_CPU_ABI_VERSION
  int32_t dtype;        // 2: fp32, 5: fp64 (the ditto_dtype codes of the HIP library)
  int32_t inter_op;     // 0 cast (nothing to do in one precision), 1 relu, 2 softmax (scale, max-subtracted, over L)
  int32_t relu_out;     // ReLU on the second accumulator (cast / relu chains)
  int64_t batch, M, N, K, L;
  int64_t a_batch_stride, a_row_stride;  // elements; rows contiguous
  int64_t b_batch_stride, b_row_stride;  // B[batch][K][L]
  int64_t c_batch_stride, c_row_stride;  // C[batch][L][N]
  int64_t f_batch_stride, f_row_stride;
  float softmax_scale;
  // the tiling of a CPUTensorizeParam (src/auto_tensorize/hyper_fusion.cc:609-642)
  int32_t mi, ni1, ni2;  // micro-kernel tile: mi rows; ni1 columns of the intermediate, ni2 of the output
  int32_t m_block;       // rows of the chain one parallel task owns (a multiple of mi)
  int32_t l_block;       // columns of the intermediate computed before the second contraction consumes them (a multiple of ni1)
  int32_t threads;       // 0: the OpenMP default
  const void* update1;   // optional micro-kernels (ditto_cpu_update_f32 / _f64) for full mi x ni1 and mi x ni2 tiles
  const void* update2;
} ditto_cpu_chain_desc;

}  // extern "C"

namespace {

thread_local char g_err[256] = "";
int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return -1;
}

// ---- built-in micro-kernels: MR x 16 fp32 on twelve ymm accumulators, MR x 8 fp64; any tile by a plain loop
template <int MR>
inline void update_f32_16(const float* a, long lda, const float* b, long ldb, float* c, long ldc, long kc) {
  __m256 acc[MR][2];
  for (int r = 0; r < MR; ++r) {
    acc[r][0] = _mm256_loadu_ps(c + r * ldc);
    acc[r][1] = _mm256_loadu_ps(c + r * ldc + 8);
  }
  for (long k = 0; k < kc; ++k) {
    const __m256 b0 = _mm256_loadu_ps(b + k * ldb), b1 = _mm256_loadu_ps(b + k * ldb + 8);
    for (int r = 0; r < MR; ++r) {
      const __m256 av = _mm256_broadcast_ss(a + r * lda + k);
      acc[r][0] = _mm256_fmadd_ps(av, b0, acc[r][0]);
      acc[r][1] = _mm256_fmadd_ps(av, b1, acc[r][1]);
    }
  }
  for (int r = 0; r < MR; ++r) {
    _mm256_storeu_ps(c + r * ldc, acc[r][0]);
    _mm256_storeu_ps(c + r * ldc + 8, acc[r][1]);
  }
}
template <int MR>
inline void update_f64_8(const double* a, long lda, const double* b, long ldb, double* c, long ldc, long kc) {
  __m256d acc[MR][2];
  for (int r = 0; r < MR; ++r) {
    acc[r][0] = _mm256_loadu_pd(c + r * ldc);
    acc[r][1] = _mm256_loadu_pd(c + r * ldc + 4);
  }
  for (long k = 0; k < kc; ++k) {
    const __m256d b0 = _mm256_loadu_pd(b + k * ldb), b1 = _mm256_loadu_pd(b + k * ldb + 4);
    for (int r = 0; r < MR; ++r) {
      const __m256d av = _mm256_broadcast_sd(a + r * lda + k);
      acc[r][0] = _mm256_fmadd_pd(av, b0, acc[r][0]);
      acc[r][1] = _mm256_fmadd_pd(av, b1, acc[r][1]);
    }
  }
  for (int r = 0; r < MR; ++r) {
    _mm256_storeu_pd(c + r * ldc, acc[r][0]);
    _mm256_storeu_pd(c + r * ldc + 4, acc[r][1]);
  }
}
template <typename T>
inline void update_any(int mr, int nr, const T* a, long lda, const T* b, long ldb, T* c, long ldc, long kc) {
  for (int r = 0; r < mr; ++r)
    for (long k = 0; k < kc; ++k) {
      const T av = a[r * lda + k];
      for (int j = 0; j < nr; ++j) c[r * ldc + j] += av * b[k * ldb + j];
    }
}
template <typename T>
struct Vec;
template <>
struct Vec<float> {
  static constexpr int kCols = 16;
  template <int MR>
  static void run(const float* a, long lda, const float* b, long ldb, float* c, long ldc, long kc) {
    update_f32_16<MR>(a, lda, b, ldb, c, ldc, kc);
  }
};
template <>
struct Vec<double> {
  static constexpr int kCols = 8;
  template <int MR>
  static void run(const double* a, long lda, const double* b, long ldb, double* c, long ldc, long kc) {
    update_f64_8<MR>(a, lda, b, ldb, c, ldc, kc);
  }
};

// c[mr][nc] += a[mr][kc] . b[kc][nc], mr <= mi, walked in tiles of ni columns: the caller's micro-kernel on full
// tiles, the built-in vector kernel on panels of its width, a plain loop on what is left
template <typename T>
void panel(int mi, int ni, void (*ext)(const T*, long, const T*, long, T*, long, long), int mr, long nc, long kc,
           const T* a, long lda, const T* b, long ldb, T* c, long ldc) {
  long j = 0;
  if (ext && mr == mi)
    for (; j + ni <= nc; j += ni) ext(a, lda, b + j, ldb, c + j, ldc, kc);
  constexpr int W = Vec<T>::kCols;
  for (; j + W <= nc; j += W) {
    switch (mr) {
      case 6: Vec<T>::template run<6>(a, lda, b + j, ldb, c + j, ldc, kc); break;
      case 5: Vec<T>::template run<5>(a, lda, b + j, ldb, c + j, ldc, kc); break;
      case 4: Vec<T>::template run<4>(a, lda, b + j, ldb, c + j, ldc, kc); break;
      case 3: Vec<T>::template run<3>(a, lda, b + j, ldb, c + j, ldc, kc); break;
      case 2: Vec<T>::template run<2>(a, lda, b + j, ldb, c + j, ldc, kc); break;
      case 1: Vec<T>::template run<1>(a, lda, b + j, ldb, c + j, ldc, kc); break;
      default: update_any<T>(mr, W, a, lda, b + j, ldb, c + j, ldc, kc);
    }
  }
  if (j < nc) update_any<T>(mr, (int)(nc - j), a, lda, b + j, ldb, c + j, ldc, kc);
}

template <typename T>
int run_chain(const ditto_cpu_chain_desc& d, const T* A, const T* B, const T* C, T* F) {
  typedef void (*Upd)(const T*, long, const T*, long, T*, long, long);
  const Upd u1 = reinterpret_cast<Upd>(const_cast<void*>(d.update1));
  const Upd u2 = reinterpret_cast<Upd>(const_cast<void*>(d.update2));
  const int mi = d.mi;
  const long M = d.M, N = d.N, K = d.K, L = d.L;
  const long mb = d.m_block, lb = d.l_block;
  const long mblocks = (M + mb - 1) / mb;
  const long tasks = d.batch * mblocks;
  const bool softmax = d.inter_op == 2;
  const T scale = (T)d.softmax_scale;
  const int nthreads = d.threads > 0 ? d.threads : omp_get_max_threads();
#pragma omp parallel num_threads(nthreads)
  {
    // per thread: the tile of the first contraction (the compute_at position of the reference's nest), the second
    // accumulator of the task's rows, and the softmax state of those rows
    std::vector<T> dt((size_t)mb * lb), ft((size_t)mb * N), rmax, rsum;
    if (softmax) rmax.resize(mb), rsum.resize(mb);
#pragma omp for schedule(dynamic, 1)
    for (long t = 0; t < tasks; ++t) {
      const long bz = t / mblocks, m0 = (t % mblocks) * mb;
      const long rows = std::min(mb, M - m0);
      const T* a = A + bz * d.a_batch_stride + m0 * d.a_row_stride;
      const T* b = B + bz * d.b_batch_stride;
      const T* c = C + bz * d.c_batch_stride;
      std::fill(ft.begin(), ft.begin() + rows * N, (T)0);
      if (softmax) {
        std::fill(rmax.begin(), rmax.begin() + rows, -std::numeric_limits<T>::infinity());
        std::fill(rsum.begin(), rsum.begin() + rows, (T)0);
      }
      for (long l0 = 0; l0 < L; l0 += lb) {
        const long lc = std::min(lb, L - l0);
        // first contraction at this position: dt[rows][lc] = a[rows][K] . b[K][l0 .. l0 + lc)
        for (long r = 0; r < rows; ++r) std::fill(dt.begin() + r * lb, dt.begin() + r * lb + lc, (T)0);
        for (long r = 0; r < rows; r += mi)
          panel<T>(mi, d.ni1, u1, (int)std::min<long>(mi, rows - r), lc, K, a + r * d.a_row_stride, d.a_row_stride,
                   b + l0, d.b_row_stride, dt.data() + r * lb, lb);
        // the op between the contractions, on the tile while it is in cache
        if (d.inter_op == 1) {
          for (long r = 0; r < rows; ++r)
            for (long j = 0; j < lc; ++j) dt[r * lb + j] = std::max(dt[r * lb + j], (T)0);
        } else if (softmax) {
          for (long r = 0; r < rows; ++r) {
            T* row = dt.data() + r * lb;
            T mx = rmax[r];
            for (long j = 0; j < lc; ++j) mx = std::max(mx, row[j] * scale);
            if (mx > rmax[r]) {  // the rows' running maximum moved: what has been summed so far shrinks with it
              const T alpha = std::exp(rmax[r] - mx);
              rsum[r] *= alpha;
              for (long n = 0; n < N; ++n) ft[r * N + n] *= alpha;
              rmax[r] = mx;
            }
            T s = 0;
            for (long j = 0; j < lc; ++j) {
              row[j] = std::exp(row[j] * scale - mx);
              s += row[j];
            }
            rsum[r] += s;
          }
        }
        // second contraction: ft[rows][N] += dt[rows][lc] . c[l0 .. l0 + lc)[N]
        for (long r = 0; r < rows; r += mi)
          panel<T>(mi, d.ni2, u2, (int)std::min<long>(mi, rows - r), N, lc, dt.data() + r * lb, lb, c + l0 * d.c_row_stride,
                   d.c_row_stride, ft.data() + r * N, N);
      }
      T* f = F + bz * d.f_batch_stride + m0 * d.f_row_stride;
      for (long r = 0; r < rows; ++r) {
        const T inv = softmax ? (T)1 / rsum[r] : (T)1;
        for (long n = 0; n < N; ++n) {
          T v = ft[r * N + n] * inv;
          if (!softmax && d.relu_out) v = std::max(v, (T)0);
          f[r * d.f_row_stride + n] = v;
        }
      }
    }
  }
  return 0;
}

}  // namespace

extern "C" {

__attribute__((visibility("default"))) int ditto_cpu_chain_abi_version(void) { return DITTO_CPU_ABI_VERSION; }
__attribute__((visibility("default"))) const char* ditto_cpu_last_error(void) { return g_err; }

// Runs the fused chain on host memory; blocking (the reference's LLVM target is, too).  0 or -1 with a message.
__attribute__((visibility("default"))) int ditto_cpu_bmm_chain_run(const ditto_cpu_chain_desc* d, const void* a,
                                                                  const void* b, const void* c, void* f) {
  if (!d || !a || !b || !c || !f) return fail("null argument");
  if (d->abi_version != DITTO_CPU_ABI_VERSION) return fail("descriptor abi_version %d, library %d", d->abi_version, DITTO_CPU_ABI_VERSION);
  if (d->dtype != 2 && d->dtype != 5) return fail("the CPU micro-kernels are fp32 / fp64 (dtype code %d)", d->dtype);
  if (d->inter_op < 0 || d->inter_op > 2) return fail("inter_op %d not valid", d->inter_op);
  if (d->batch <= 0 || d->M <= 0 || d->N <= 0 || d->K <= 0 || d->L <= 0) return fail("extents must be positive");
  if (d->a_row_stride < d->K || d->b_row_stride < d->L || d->c_row_stride < d->N || d->f_row_stride < d->N)
    return fail("row stride smaller than row extent");
  if (d->mi < 1 || d->mi > 6) return fail("micro-kernel rows mi = %d: 1 .. 6", d->mi);
  if (d->ni1 < 1 || d->ni2 < 1) return fail("micro-kernel columns must be positive");
  if (d->m_block < d->mi || d->m_block % d->mi) return fail("m_block %d must be a positive multiple of mi %d", d->m_block, d->mi);
  if (d->l_block < 1) return fail("l_block must be positive");
  if (d->inter_op == 2 && !(d->softmax_scale > 0)) return fail("softmax_scale must be > 0");
  if (d->dtype == 2)
    return run_chain<float>(*d, static_cast<const float*>(a), static_cast<const float*>(b), static_cast<const float*>(c),
                            static_cast<float*>(f));
  return run_chain<double>(*d, static_cast<const double*>(a), static_cast<const double*>(b), static_cast<const double*>(c),
                           static_cast<double*>(f));
}

}  // extern "C"
