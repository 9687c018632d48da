/*
 * chain_oracle.c -- CPU restatement of Ditto's fused operator chains.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP kernels: it is
 * built into oracle/libchain_oracle.so and called from tests/, from
 * __graft_entry__.smoke() and from the cpu_baseline leg of bench.py.  Nothing in the
 * product package (ditto_amd/) imports, links or executes it.
 *
 * What is restated (the reference computes these through TVM-generated code, which
 * cannot be built here: 3rdparty/tvm is an empty submodule):
 *
 *   oracle_bmm_chain_f64      closed form of  F = epi(inter(A.B).C)  in double; the
 *                             chain semantics of benchmark/chimera/cuda/bmm_bmm_cuda.py:69-149
 *                             (cast chain) and python/ditto/auto_compute/nn/functional/
 *                             bmm_chain.py:5-105 (softmax chain), with the roundings of
 *                             the intermediate and the output to in_dtype made explicit.
 *   oracle_bmm_chain_fused_f32  the fused CPU loop nest of TensorizeCPU
 *                             (src/auto_tensorize/hyper_fusion_cpu.cc:644-907): the outer
 *                             loops of the second contraction are split and run in
 *                             parallel, the first contraction is computed at the second
 *                             one's last common loop into a cache-resident tile, and both
 *                             use a 6x16 fp32 register tile
 *                             (python/ditto/auto_tensorize/intrinsic.py:292-416).
 *   oracle_bmm_softmax_ref_emul  the reference's own softmax form: exp without max
 *                             subtraction, row sum obtained from a column of ones appended
 *                             to the second operand, final divide with +1e-5
 *                             (bmm_chain.py:63-103).
 *   oracle_gemm_chain_i8      exact integer chain with the middle result requantised to
 *                             int8 (round to nearest even, saturate to [-128,127]).  The
 *                             requantise step is NOT in the reference (its int8 chain does a
 *                             wrapping astype("int8"), bmm_bmm_cuda.py:116): it is specified
 *                             by this build's workload definition.
 *   oracle_gemm_chain_i8_wrap the reference's own int8 chain: the int32 middle result goes back to
 *                             int8 with astype("int8"), which keeps the low byte (two's complement
 *                             wrap), optionally behind a ReLU (bmm_bmm_cuda.py:114-118).
 *   oracle_conv_chain_grouped_f32  the same with a grouped (depthwise) first convolution
 *   oracle_conv_chain_f32     conv -> inter -> conv on NCHW tensors, the chain of
 *                             benchmark/chimera/cuda/conv3x3_conv1x1_cuda.py:77-172 in the
 *                             plain layout of testing/hyper_fusion/
 *                             conv_relu_conv_relu_fuse_hw_cuda.py:17-262.
 *
 * Pinning (tests/test_oracle.py): every function is checked against numpy/torch closed
 * forms, brute-force loops on tiny shapes, and algebraic invariants (identity operand,
 * linearity, softmax shift invariance, delta-kernel convolution, integer vs float
 * requantise formula).  The reference holds no golden vectors for this path.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORACLE_API __attribute__((visibility("default")))

/* rounding of an fp32 value to the value set of a narrower type, returned as fp32 */
enum { ROUND_NONE = 0, ROUND_F16 = 1, ROUND_BF16 = 2, ROUND_F32 = 3 };
/* op between the two contractions */
enum { INTER_CAST = 0, INTER_RELU = 1, INTER_SOFTMAX = 2 };

static inline uint32_t f2u(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float u2f(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

/* fp32 -> bf16 -> fp32, round to nearest even; NaN stays NaN */
ORACLE_API float oracle_round_bf16(float x) {
  uint32_t u = f2u(x);
  if ((u & 0x7fffffffu) > 0x7f800000u) return u2f(u | 0x00400000u);
  uint32_t lsb = (u >> 16) & 1u;
  u += 0x7fffu + lsb;
  return u2f(u & 0xffff0000u);
}

/* fp32 -> fp16 -> fp32, round to nearest even, IEEE binary16 with subnormals and
 * overflow to infinity */
ORACLE_API float oracle_round_f16(float x) {
  uint32_t u = f2u(x);
  uint32_t sign = u & 0x80000000u;
  uint32_t a = u & 0x7fffffffu;
  if (a >= 0x7f800000u) return x; /* inf / nan */
  if (a >= 0x477ff000u) {         /* >= 65520 rounds to inf */
    return u2f(sign | 0x7f800000u);
  }
  if (a < 0x38800000u) { /* below the smallest normal half, 2^-14: subnormal spacing 2^-24 */
    float ax = u2f(a);
    /* adding and subtracting 0.5 = 2^-1 * ... : use the magic constant 2^(23-24) trick:
       ax + 2^-1 ... ; spacing 2^-24 is the ulp of values in [2^-1, 2^0) */
    float magic = 0.5f;
    float r = (ax + magic) - magic; /* RNE to a multiple of 2^-24 under default rounding */
    return u2f(sign | f2u(r));
  }
  uint32_t lsb = (a >> 13) & 1u;
  a += 0xfffu + lsb;
  a &= 0xffffe000u;
  return u2f(sign | a);
}

static inline float round_to(float x, int mode) {
  if (mode == ROUND_F16) return oracle_round_f16(x);
  if (mode == ROUND_BF16) return oracle_round_bf16(x);
  return x;
}

/* rounding of a double intermediate: ROUND_NONE keeps it in double */
static inline double round_to_d(double x, int mode) {
  if (mode == ROUND_NONE) return x;
  return (double)round_to((float)x, mode);
}

ORACLE_API void oracle_round_array(const float* x, float* y, long long n, int mode) {
  for (long long i = 0; i < n; ++i) y[i] = round_to(x[i], mode);
}

/* ------------------------------------------------------------------------------------
 * Closed form in double.  A[b][M][K], B[b][K][L], C[b][L][N] row-major fp32 arrays (the
 * caller has already rounded them to in_dtype), F[b][M][N].
 *   inter = CAST   : mid = round_in(A.B)
 *   inter = RELU   : mid = round_in(max(A.B, 0))          (conv_relu..._cuda.py:134-142
 *                                                           compares the accumulator)
 *   inter = SOFTMAX: mid = softmax_L(scale * A.B), max-subtracted, NOT rounded
 * F = round_out(mid . C).  round_mid / round_out select the rounding (ROUND_*;
 * ROUND_NONE keeps the intermediate in double, ROUND_F32 rounds it to fp32).
 * ---------------------------------------------------------------------------------- */
ORACLE_API void oracle_bmm_chain_f64(int batch, int M, int N, int K, int L, const float* A,
                                     const float* B, const float* C, float* F, int inter,
                                     double scale, int round_mid, int round_out) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < batch; ++b) {
    for (int m = 0; m < M; ++m) {
      double* mid = (double*)malloc(sizeof(double) * (size_t)L);
      const float* a = A + ((size_t)b * M + m) * K;
      const float* Bb = B + (size_t)b * K * L;
      const float* Cb = C + (size_t)b * L * N;
      for (int l = 0; l < L; ++l) {
        double acc = 0.0;
        for (int k = 0; k < K; ++k) acc += (double)a[k] * (double)Bb[(size_t)k * L + l];
        mid[l] = acc;
      }
      if (inter == INTER_SOFTMAX) {
        double mx = -INFINITY, sum = 0.0;
        for (int l = 0; l < L; ++l) mx = fmax(mx, mid[l] * scale);
        for (int l = 0; l < L; ++l) {
          mid[l] = exp(mid[l] * scale - mx);
          sum += mid[l];
        }
        for (int l = 0; l < L; ++l) mid[l] /= sum;
      } else {
        for (int l = 0; l < L; ++l) {
          double v = mid[l];
          if (inter == INTER_RELU && v < 0.0) v = 0.0;
          mid[l] = round_to_d(v, round_mid);
        }
      }
      float* f = F + ((size_t)b * M + m) * N;
      for (int n = 0; n < N; ++n) {
        double acc = 0.0;
        for (int l = 0; l < L; ++l) acc += mid[l] * (double)Cb[(size_t)l * N + n];
        f[n] = round_to((float)acc, round_out);
      }
      free(mid);
    }
  }
}

/* ------------------------------------------------------------------------------------
 * The reference's softmax chain, op by op (bmm_chain.py:40-103):
 *   D = A.B (fp32 acc) ; P = round_in(exp(D)) ; E = P.[C | 1] (fp32 acc; the ones column
 *   yields the row sum) ; F = round_in( round_in(E[m][n]) / (round_in(E[m][sum]) + 1e-5) )
 * No scale and no max subtraction: exp overflows the narrow type for scores above ~11
 * (fp16), which is why the reference only feeds it uniform(-1,1) inputs.
 * ---------------------------------------------------------------------------------- */
ORACLE_API void oracle_bmm_softmax_ref_emul(int batch, int M, int N, int K, int L, const float* A,
                                            const float* B, const float* C, float* F,
                                            int round_in) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < batch; ++b) {
    for (int m = 0; m < M; ++m) {
      float* p = (float*)malloc(sizeof(float) * (size_t)L);
      const float* a = A + ((size_t)b * M + m) * K;
      const float* Bb = B + (size_t)b * K * L;
      const float* Cb = C + (size_t)b * L * N;
      for (int l = 0; l < L; ++l) {
        float acc = 0.f;
        for (int k = 0; k < K; ++k) acc += a[k] * Bb[(size_t)k * L + l];
        p[l] = round_to(expf(acc), round_in);
      }
      float den = 0.f;
      for (int l = 0; l < L; ++l) den += p[l];
      const float eps = round_to(1e-5f, round_in);
      const float denr = round_to(round_to(den, round_in) + eps, round_in);
      float* f = F + ((size_t)b * M + m) * N;
      for (int n = 0; n < N; ++n) {
        float acc = 0.f;
        for (int l = 0; l < L; ++l) acc += p[l] * Cb[(size_t)l * N + n];
        f[n] = round_to(round_to(acc, round_in) / denr, round_in);
      }
      free(p);
    }
  }
}

/* ------------------------------------------------------------------------------------
 * Fused CPU loop nest (TensorizeCPU, hyper_fusion_cpu.cc:644-907).
 *
 * 6x16 register tile, broadcast-FMA over the reduce axis (intrinsic.py:341-366): for each
 * k, one 16-wide row of the right operand is multiplied by 6 broadcast scalars of the left
 * operand.  Left operand rows beyond `mr` (< 6) and right columns beyond `nr` (< 16) are
 * skipped, which is what the reference's zero padding to multiples of 6 / 16 achieves
 * (bmm_softmax_bmm.py:67-100).
 * ---------------------------------------------------------------------------------- */
#define MI 6
#define NI 16

static inline void micro_6x16(int kc, const float* a, int lda, const float* b, int ldb, float* c,
                              int ldc, int mr, int nr, int accumulate) {
  float acc[MI][NI];
  for (int i = 0; i < MI; ++i)
    for (int j = 0; j < NI; ++j) acc[i][j] = 0.f;
  if (mr == MI && nr == NI) {
    for (int k = 0; k < kc; ++k) {
      const float* brow = b + (size_t)k * ldb;
      for (int i = 0; i < MI; ++i) {
        const float av = a[(size_t)i * lda + k];
#pragma omp simd
        for (int j = 0; j < NI; ++j) acc[i][j] += av * brow[j];
      }
    }
  } else {
    for (int k = 0; k < kc; ++k) {
      const float* brow = b + (size_t)k * ldb;
      for (int i = 0; i < mr; ++i) {
        const float av = a[(size_t)i * lda + k];
        for (int j = 0; j < nr; ++j) acc[i][j] += av * brow[j];
      }
    }
  }
  for (int i = 0; i < mr; ++i)
    for (int j = 0; j < nr; ++j) {
      if (accumulate)
        c[(size_t)i * ldc + j] += acc[i][j];
      else
        c[(size_t)i * ldc + j] = acc[i][j];
    }
}

/* C[mc x nc] (+)= A[mc x kc] . B[kc x nc] with the 6x16 micro-kernel */
static void tile_gemm(int mc, int nc, int kc, const float* a, int lda, const float* b, int ldb,
                      float* c, int ldc, int accumulate) {
  for (int i = 0; i < mc; i += MI) {
    const int mr = mc - i < MI ? mc - i : MI;
    for (int j = 0; j < nc; j += NI) {
      const int nr = nc - j < NI ? nc - j : NI;
      micro_6x16(kc, a + (size_t)i * lda, lda, b + j, ldb, c + (size_t)i * ldc + j, ldc, mr, nr,
                 accumulate);
    }
  }
}

/*
 * Fused nest: parallel over (batch x M blocks of `mb` rows); inside, the second
 * contraction's reduce axis L is the common loop, walked in tiles of `lb`: the first
 * contraction produces mid[mb x lb] into a per-thread buffer (compute_at the common loop,
 * hyper_fusion_cpu.cc:813-814), the inter op is applied in place, and the second
 * contraction accumulates E[mb x N] from it.
 *   CAST/RELU: any lb.  SOFTMAX: the whole row block [mb x L] is produced first (lb = L),
 *   max-subtracted exp and row sum are taken, then E = P.C is divided by the sum
 *   (the CPU form of the reference divides by the ones-column, bmm_softmax_bmm.py:148-166).
 * mb is rounded to a multiple of 6.  Returns 0, or -1 if a buffer cannot be allocated.
 */
ORACLE_API int oracle_bmm_chain_fused_f32(int batch, int M, int N, int K, int L, const float* A,
                                          const float* B, const float* C, float* F, int inter,
                                          float scale, int round_mid, int round_out, int mb,
                                          int lb, int threads) {
  if (mb < MI) mb = MI;
  mb = (mb / MI) * MI;
  if (lb < NI) lb = NI;
  if (inter == INTER_SOFTMAX) lb = L;
  if (lb > L) lb = L;
  const int mblocks = (M + mb - 1) / mb;
  int failed = 0;
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#else
  (void)threads;
#endif
#pragma omp parallel
  {
    float* mid = (float*)malloc(sizeof(float) * (size_t)mb * lb);
    float* E = (float*)malloc(sizeof(float) * (size_t)mb * N);
    float* rsum = (float*)malloc(sizeof(float) * (size_t)mb);
    if (!mid || !E || !rsum) {
#pragma omp atomic write
      failed = 1;
    } else {
#pragma omp for collapse(2) schedule(dynamic, 1)
      for (int b = 0; b < batch; ++b) {
        for (int blk = 0; blk < mblocks; ++blk) {
          const int m0 = blk * mb;
          const int mc = M - m0 < mb ? M - m0 : mb;
          const float* Ab = A + ((size_t)b * M + m0) * K;
          const float* Bb = B + (size_t)b * K * L;
          const float* Cb = C + (size_t)b * L * N;
          for (int l0 = 0; l0 < L; l0 += lb) {
            const int lc = L - l0 < lb ? L - l0 : lb;
            /* first contraction at the common loop */
            tile_gemm(mc, lc, K, Ab, K, Bb + l0, L, mid, lb, 0);
            /* inter path, in place */
            if (inter == INTER_SOFTMAX) {
              for (int i = 0; i < mc; ++i) {
                float* row = mid + (size_t)i * lb;
                float mx = -INFINITY;
                for (int l = 0; l < lc; ++l) {
                  row[l] *= scale;
                  mx = row[l] > mx ? row[l] : mx;
                }
                float s = 0.f;
                for (int l = 0; l < lc; ++l) {
                  row[l] = expf(row[l] - mx);
                  s += row[l];
                }
                rsum[i] = s;
                if (round_mid != ROUND_NONE)
                  for (int l = 0; l < lc; ++l) row[l] = round_to(row[l], round_mid);
              }
            } else {
              for (int i = 0; i < mc; ++i) {
                float* row = mid + (size_t)i * lb;
                for (int l = 0; l < lc; ++l) {
                  float v = row[l];
                  if (inter == INTER_RELU && v < 0.f) v = 0.f;
                  row[l] = round_to(v, round_mid);
                }
              }
            }
            /* second contraction */
            tile_gemm(mc, N, lc, mid, lb, Cb + (size_t)l0 * N, N, E, N, l0 != 0);
          }
          for (int i = 0; i < mc; ++i) {
            float* f = F + ((size_t)b * M + m0 + i) * N;
            const float inv = inter == INTER_SOFTMAX ? 1.f / rsum[i] : 1.f;
            for (int n = 0; n < N; ++n) f[n] = round_to(E[(size_t)i * N + n] * inv, round_out);
          }
        }
      }
    }
    free(mid);
    free(E);
    free(rsum);
  }
  return failed ? -1 : 0;
}

/* ------------------------------------------------------------------------------------
 * int8 chain:  mid = A.B (int32) ; q = sat_i8(rne(mid * scale[l])) ; E = q.D (int32).
 * A[M][K], B[K][L], D[L][N] int8, scale[L] fp32, E[M][N] int32.
 * The requantise arithmetic is fp32: (float)mid is exact for |mid| < 2^24, the product is
 * one IEEE multiply, rintf rounds to nearest even, then clamp to [-128,127].
 * ---------------------------------------------------------------------------------- */
static inline int8_t requant_f32(int32_t mid, float s) {
  float v = rintf((float)mid * s);
  if (v > 127.f) v = 127.f;
  if (v < -128.f) v = -128.f;
  return (int8_t)(int32_t)v;
}

/* the same step for a power-of-two scale 2^-shift in pure integer arithmetic */
ORACLE_API int32_t oracle_requant_shift(int32_t mid, int shift) {
  int64_t q;
  if (shift <= 0) {
    q = (int64_t)mid << (-shift);
  } else {
    const int64_t q0 = (int64_t)mid >> shift; /* arithmetic shift = floor */
    const int64_t r = (int64_t)mid & (((int64_t)1 << shift) - 1);
    const int64_t half = (int64_t)1 << (shift - 1);
    q = q0 + ((r > half) || (r == half && (q0 & 1)));
  }
  if (q > 127) q = 127;
  if (q < -128) q = -128;
  return (int32_t)q;
}

ORACLE_API int32_t oracle_requant_scale(int32_t mid, float s) { return (int32_t)requant_f32(mid, s); }

/* E = wrap_i8(relu?(A.B)) . D in exact integers (bmm_bmm_cuda.py:114-118: astype("int8") of the int32 product). */
ORACLE_API void oracle_gemm_chain_i8_wrap(int batch, int M, int N, int K, int L, const int8_t* A,
                                          const int8_t* B, const int8_t* D, int relu, int32_t* E,
                                          int8_t* mid_out) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < batch; ++b) {
    for (int m = 0; m < M; ++m) {
      int32_t* mid = (int32_t*)calloc((size_t)L, sizeof(int32_t));
      int8_t* q = (int8_t*)malloc((size_t)L);
      const int8_t* a = A + ((size_t)b * M + m) * K;
      const int8_t* Bb = B + (size_t)b * K * L;
      const int8_t* Db = D + (size_t)b * L * N;
      for (int k = 0; k < K; ++k) {
        const int32_t av = a[k];
        const int8_t* brow = Bb + (size_t)k * L;
        for (int l = 0; l < L; ++l) mid[l] += av * (int32_t)brow[l];
      }
      for (int l = 0; l < L; ++l) {
        int32_t v = mid[l];
        if (relu && v < 0) v = 0;
        const uint32_t low = (uint32_t)v & 0xffu; /* the low byte, read back as a signed 8-bit value */
        q[l] = (int8_t)(low >= 128u ? (int32_t)low - 256 : (int32_t)low);
      }
      if (mid_out) memcpy(mid_out + ((size_t)b * M + m) * L, q, (size_t)L);
      int32_t* e = E + ((size_t)b * M + m) * N;
      for (int n = 0; n < N; ++n) e[n] = 0;
      for (int l = 0; l < L; ++l) {
        const int32_t qv = q[l];
        const int8_t* drow = Db + (size_t)l * N;
        for (int n = 0; n < N; ++n) e[n] += qv * (int32_t)drow[n];
      }
      free(mid);
      free(q);
    }
  }
}

ORACLE_API void oracle_gemm_chain_i8(int batch, int M, int N, int K, int L, const int8_t* A,
                                     const int8_t* B, const int8_t* D, const float* scale,
                                     int32_t* E, int8_t* mid_out) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int b = 0; b < batch; ++b) {
    for (int m = 0; m < M; ++m) {
      int32_t* mid = (int32_t*)calloc((size_t)L, sizeof(int32_t));
      int8_t* q = (int8_t*)malloc((size_t)L);
      const int8_t* a = A + ((size_t)b * M + m) * K;
      const int8_t* Bb = B + (size_t)b * K * L;
      const int8_t* Db = D + (size_t)b * L * N;
      for (int k = 0; k < K; ++k) {
        const int32_t av = a[k];
        const int8_t* brow = Bb + (size_t)k * L;
        for (int l = 0; l < L; ++l) mid[l] += av * (int32_t)brow[l];
      }
      for (int l = 0; l < L; ++l) q[l] = requant_f32(mid[l], scale[l]);
      if (mid_out) memcpy(mid_out + ((size_t)b * M + m) * L, q, (size_t)L);
      int32_t* e = E + ((size_t)b * M + m) * N;
      for (int n = 0; n < N; ++n) e[n] = 0;
      for (int l = 0; l < L; ++l) {
        const int32_t qv = q[l];
        const int8_t* drow = Db + (size_t)l * N;
        for (int n = 0; n < N; ++n) e[n] += qv * (int32_t)drow[n];
      }
      free(mid);
      free(q);
    }
  }
}

/* ------------------------------------------------------------------------------------
 * conv -> inter -> conv, NCHW.  X[N][C0][H][W], W1[C1][C0][R1][S1], W2[C2][C1][R2][S2],
 * Y[N][C2][P2][Q2]; fp32 accumulation; the intermediate is rounded to in_dtype
 * (conv3x3_conv1x1_cuda.py:132-136) after an optional ReLU on the accumulator, the output
 * is rounded to out dtype after an optional ReLU.  `mid` is caller-provided scratch of
 * N*C1*P1*Q1 floats.
 * ---------------------------------------------------------------------------------- */
/* groups: input channels and output channels are split into `groups` equal parts and output
 * channel k only sees the inputs of its part (groups = C: depthwise, Kc / C outputs per input
 * channel; weights [Kc][C / groups][R][S]) */
static void conv2d_nchw(int N, int C, int H, int W, int Kc, int R, int S, int pad, int stride, int groups,
                        const float* x, const float* w, float* y, int relu, int round_mode) {
  const int cg = C / groups, kg = Kc / groups;
  const int P = (H + 2 * pad - R) / stride + 1;
  const int Q = (W + 2 * pad - S) / stride + 1;
#pragma omp parallel for collapse(2) schedule(static)
  for (int n = 0; n < N; ++n) {
    for (int k = 0; k < Kc; ++k) {
      float* yp = y + ((size_t)n * Kc + k) * P * Q;
      for (int i = 0; i < P * Q; ++i) yp[i] = 0.f;
      for (int ci = 0; ci < cg; ++ci) {
        const int c = (k / kg) * cg + ci;
        const float* xp = x + ((size_t)n * C + c) * H * W;
        const float* wp = w + ((size_t)k * cg + ci) * R * S;
        for (int r = 0; r < R; ++r)
          for (int s = 0; s < S; ++s) {
            const float wv = wp[r * S + s];
            for (int p = 0; p < P; ++p) {
              const int h = p * stride + r - pad;
              if (h < 0 || h >= H) continue;
              /* q range with 0 <= q*stride + s - pad < W */
              int q_lo = 0;
              while (q_lo < Q && q_lo * stride + s - pad < 0) ++q_lo;
              int q_hi = Q;
              while (q_hi > q_lo && (q_hi - 1) * stride + s - pad >= W) --q_hi;
              const float* xrow = xp + (size_t)h * W + (s - pad);
              float* yrow = yp + (size_t)p * Q;
              for (int q = q_lo; q < q_hi; ++q) yrow[q] += wv * xrow[q * stride];
            }
          }
      }
      for (int i = 0; i < P * Q; ++i) {
        float v = yp[i];
        if (relu && v < 0.f) v = 0.f;
        yp[i] = round_to(v, round_mode);
      }
    }
  }
}

ORACLE_API void oracle_conv_chain_f32(int N, int C0, int H, int W, int C1, int R1, int S1, int pad1,
                                      int stride1, int C2, int R2, int S2, int pad2, int stride2,
                                      const float* X, const float* W1, const float* W2, float* mid,
                                      float* Y, int relu_mid, int relu_out, int round_mid,
                                      int round_out) {
  const int P1 = (H + 2 * pad1 - R1) / stride1 + 1;
  const int Q1 = (W + 2 * pad1 - S1) / stride1 + 1;
  conv2d_nchw(N, C0, H, W, C1, R1, S1, pad1, stride1, 1, X, W1, mid, relu_mid, round_mid);
  conv2d_nchw(N, C1, P1, Q1, C2, R2, S2, pad2, stride2, 1, mid, W2, Y, relu_out, round_out);
}

/* the same chain with a grouped first convolution (groups1 = C0: the depthwise -> 1x1 chain of
 * benchmark/chimera/cuda/depthwise3x3_conv1x1_small_channel_cuda.py:77-169, whose `factor` is
 * C1 / C0) */
ORACLE_API void oracle_conv_chain_grouped_f32(int N, int C0, int H, int W, int C1, int R1, int S1, int pad1,
                                              int stride1, int groups1, int C2, int R2, int S2, int pad2,
                                              int stride2, const float* X, const float* W1, const float* W2,
                                              float* mid, float* Y, int relu_mid, int relu_out, int round_mid,
                                              int round_out) {
  const int P1 = (H + 2 * pad1 - R1) / stride1 + 1;
  const int Q1 = (W + 2 * pad1 - S1) / stride1 + 1;
  conv2d_nchw(N, C0, H, W, C1, R1, S1, pad1, stride1, groups1, X, W1, mid, relu_mid, round_mid);
  conv2d_nchw(N, C1, P1, Q1, C2, R2, S2, pad2, stride2, 1, mid, W2, Y, relu_out, round_out);
}

ORACLE_API int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
