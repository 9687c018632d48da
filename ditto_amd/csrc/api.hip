// C ABI of the chain library: descriptor validation, tile choice, kernel dispatch.
// Declarations and the reference interfaces they replace are in include/ditto_chain.h.
#include "../../include/ditto_chain.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <vector>

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

#include "bmm_chain_fp8.h"
#include "bmm_chain_fp8m16.h"
#include "bmm_chain_fp4m16.h"
#include "chain_kernels.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// Number of compute units of the current device (cached per thread).
int device_cus() {
  static thread_local int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
      cus = prop.multiProcessorCount;
    if (cus <= 0) cus = 256;
  }
  return cus;
}

struct BmmPlan {
  int family;  // 0: fp16/bf16 register-resident chain, 1: fp32 chain, 2: int8 requant chain
  int d_pad, qt;  // fp chains: head pad and rows-per-wave code; int8 chain: row tiles and ring depth
  int nb3 = 0, nb = 0;  // 16x16x32-MFMA kernel: row blocks of 384 rows / row blocks in all, per batch entry
  ditto_tile_param tile;
};

// Row blocks of 384 and of 256 rows for the kernel on the 16x16x32 MFMA.  A 384-row workgroup does half as much
// work again as a 256-row one in about kBig3 of its time, but 384 seldom divides the rows evenly over the compute
// units: every split (a blocks of 384, then blocks of 256 for the rest) is priced by dealing its workgroups out the
// way the hardware does (an XCD takes the large blocks of all of its batch entries first, then the small ones, each
// to the compute unit that is free first) and the shortest finish wins.  Returns a.
constexpr double kBig3 = 1.43;
int plan_rows_384(long long M, long long batch, int cus) {
  thread_local long long last_m = -1, last_batch = -1;
  thread_local int last_cus = -1, last_a = 0;
  if (M == last_m && batch == last_batch && cus == last_cus) return last_a;
  const long long amax = M / 384 + (M % 384 > 256 ? 1 : 0);
  const bool split = batch % 8 == 0 && cus % 8 == 0;
  const long long per = split ? batch / 8 : batch;
  const int cu = split ? cus / 8 : cus;
  int best_a = 0;
  if (amax > 0 && per * (M / 256 + 2) > 4096) {
    best_a = (int)(M / 384);  // so many workgroups that the finish does not matter
  } else if (amax > 0) {
    double best = 0;
    std::vector<double> free_at(cu);
    for (long long a = 0; a <= amax; ++a) {
      if (a > 0 && a < amax - 16) continue;  // the finish is tuned by the last few blocks
      const long long rest = M - 384 * a;
      const long long b = rest > 0 ? (rest + 255) / 256 : 0;
      std::fill(free_at.begin(), free_at.end(), 0.0);
      auto deal = [&](long long n, double cost) {
        for (long long i = 0; i < n; ++i) *std::min_element(free_at.begin(), free_at.end()) += cost;
      };
      deal(per * a, kBig3);
      deal(per * b, 1.0);
      const double finish = *std::max_element(free_at.begin(), free_at.end());
      if (a == 0 || finish < best - 1e-9) best = finish, best_a = (int)a;
    }
  }
  last_m = M, last_batch = batch, last_cus = cus, last_a = best_a;
  return best_a;
}

int plan_bmm(const ditto_bmm_chain_desc* d, BmmPlan* plan, bool need_device) {
  if (!d) return fail(DITTO_EINVAL, "null descriptor");
  if (d->abi_version != DITTO_CHAIN_ABI_VERSION)
    return fail(DITTO_EINVAL, "descriptor abi_version %d, library %d", d->abi_version,
                DITTO_CHAIN_ABI_VERSION);
  if (d->relu_out != 0 && d->relu_out != 1) return fail(DITTO_EINVAL, "relu_out must be 0 or 1");
  if (d->relu_out && (d->in_dtype == DITTO_I8 || d->inter_op == DITTO_INTER_SOFTMAX))
    return fail(DITTO_EUNSUPPORTED, "relu_out is implemented for the cast / relu chains on fp16, bf16 and fp32");
  if (d->tile_variant < 0) return fail(DITTO_EINVAL, "tile_variant must be 0 or a variant id");
  if (d->batch_inner < 0 || (d->batch_inner > 0 && d->batch > 0 && d->batch % d->batch_inner != 0))
    return fail(DITTO_EINVAL, "batch_inner must be 0 or divide batch");
  const bool two_level = d->batch_inner > 0 && d->batch_inner != d->batch;
  if (two_level && d->in_dtype != DITTO_F16 && d->in_dtype != DITTO_BF16)
    return fail(DITTO_EUNSUPPORTED, "two-level batch strides are implemented for the fp16/bf16 chains");
  if (d->batch <= 0 || d->M <= 0 || d->N <= 0 || d->K <= 0 || d->L <= 0)
    return fail(DITTO_EINVAL, "batch, M, N, K, L must be positive (got %lld %lld %lld %lld %lld)",
                (long long)d->batch, (long long)d->M, (long long)d->N, (long long)d->K,
                (long long)d->L);
  if (d->M > 0x7fffffff / 2 || d->L > 0x7fffffff / 2 || d->batch > 0x7fffffff / 2)
    return fail(DITTO_EINVAL, "extent too large");
  if (d->b_layout != DITTO_B_KL && d->b_layout != DITTO_B_LK)
    return fail(DITTO_EINVAL, "unknown b_layout %d", d->b_layout);
  const int in = d->in_dtype;
  memset(plan, 0, sizeof(*plan));

  if (in == DITTO_F16 || in == DITTO_BF16) {
    // (an fp16 accumulator asked for with fp16 operands -- the reference's ("80", "float16", "float16") row -- is
    // served by the MFMA's fp32 accumulator: the precision asked for and more)
    if (d->acc_dtype != DITTO_F32 && !(d->acc_dtype == DITTO_F16 && in == DITTO_F16))
      return fail(DITTO_EUNSUPPORTED, "fp16/bf16 chains accumulate in fp32 (acc_dtype %d)", d->acc_dtype);
    if (d->out_dtype != in && d->out_dtype != DITTO_F32)
      return fail(DITTO_EINVAL, "out_dtype must be in_dtype or fp32");
    if (d->inter_op != DITTO_INTER_CAST && d->inter_op != DITTO_INTER_RELU &&
        d->inter_op != DITTO_INTER_SOFTMAX)
      return fail(DITTO_EINVAL, "inter_op %d not valid for a floating-point chain", d->inter_op);
    if (d->inter_op == DITTO_INTER_SOFTMAX && !(d->softmax_scale > 0.f))
      return fail(DITTO_EINVAL, "softmax_scale must be > 0");
    // 16-byte vector loads: extents and strides in multiples of 8 elements.
    // (The reference builders require multiples of 16: bmm_chain.py:34-38.)
    if (d->K % 8 || d->N % 8) return fail(DITTO_EINVAL, "K and N must be multiples of 8");
    if (d->b_layout == DITTO_B_KL && d->L % 8)
      return fail(DITTO_EINVAL, "L must be a multiple of 8 when B is [K][L]");
    if (d->a_row_stride % 8 || d->b_row_stride % 8 || d->c_row_stride % 8 || d->a_batch_stride % 8 ||
        d->b_batch_stride % 8 || d->c_batch_stride % 8)
      return fail(DITTO_EINVAL, "input strides must be multiples of 8 elements");
    if (two_level && (d->a_batch_stride_outer % 8 || d->b_batch_stride_outer % 8 || d->c_batch_stride_outer % 8 ||
                      d->f_batch_stride_outer % 4))
      return fail(DITTO_EINVAL, "outer batch strides must be multiples of 8 (inputs) / 4 (output) elements");
    const int out_vec = 4;
    if (d->f_row_stride % out_vec || d->f_batch_stride % out_vec)
      return fail(DITTO_EINVAL, "output strides must be multiples of 4 elements");
    if (d->a_row_stride < d->K || d->c_row_stride < d->N || d->f_row_stride < d->N ||
        d->b_row_stride < (d->b_layout == DITTO_B_KL ? d->L : d->K))
      return fail(DITTO_EINVAL, "row stride smaller than row extent");
    if (d->a_row_stride > 0x7fffffff || d->b_row_stride > 0x7fffffff ||
        d->c_row_stride > 0x7fffffff || d->f_row_stride > 0x7fffffff)
      return fail(DITTO_EINVAL, "row stride too large");
    // one batch entry of B and of C is addressed through a 32-bit buffer offset
    {
      const long long b_rows = d->b_layout == DITTO_B_KL ? d->K : d->L;
      if (b_rows * d->b_row_stride * 2 >= 0x7fffffffLL || d->L * d->c_row_stride * 2 >= 0x7fffffffLL)
        return fail(DITTO_EUNSUPPORTED, "a batch entry of B or C exceeds 2 GiB");
    }
    const long long dmax = d->K > d->N ? d->K : d->N;
    if (dmax > 128)
      return fail(DITTO_EUNSUPPORTED, "max(K,N)=%lld: register-resident chain supports up to 128", dmax);
    plan->family = 0;
    plan->d_pad = dmax <= 64 ? 64 : 128;
    const int cus = need_device ? device_cus() : 256;
    // Variant table (measured on MI355X, fp16 and bf16, head_pad 64 and 128).  n8 = number of 256-row
    // workgroups.  Below 3/4 of the CUs the four-wave kernel with 128-row workgroups spreads over more
    // CUs.  From there on eight waves (two per SIMD) win, in their software-pipelined form (9) at every
    // size measured.  Once there are two workgroups per CU the chip runs at its power limit and the
    // kernel on the 16x16x32 MFMA (6), which needs less energy per flop, is ahead
    // (64 x 4096 x 4096 x 128 bf16: 464 vs 484 us with the softmax, 410 vs 443 us without); at
    // head_pad 64 the pipelined kernel stays (32 x 4096 x 4096 x 64 without softmax 127.9 vs 130.0 us).
    // With B stored [K][L] (B fragments through transposing reads on the 16x16x32 kernel) the softmax at
    // head_pad 128 goes the same way (bf16 441 vs 503 us, fp16 482 vs 538), without softmax the four-wave,
    // 256-row kernel stays (431 vs 430 us).
    const long long n8 = ((d->M + 255) / 256) * d->batch;
    const bool sm = d->inter_op == DITTO_INTER_SOFTMAX;
    if (n8 >= 2LL * cus) {
      if (d->b_layout == DITTO_B_LK)
        plan->qt = plan->d_pad == 64 ? 9 : 6;
      else
        plan->qt = sm ? (plan->d_pad == 64 ? 9 : 6) : 2;
    } else if (n8 * 4 >= 3LL * cus) {
      plan->qt = 9;
    } else {
      plan->qt = 1;
    }
    // Head size up to 64: the four-wave kernels with 64-row workgroups (4: a wave owns 16 rows and all keys; 5: 32
    // rows and half the keys of every tile, half the LDS reads per MFMA for a merge at the end, ahead from 1024 keys
    // on).  Measured, fp16 and bf16, us per launch in a graph replay, best other variant -> best of 4 | 5, B stored
    // [L][K]: softmax 96 x 512 x 512 13.2 -> 11.5, 12 x 512 x 512 9.9 -> 6.9, 8 x 1024 x 1024 15.5 -> 9.9,
    // 16 x 512 x 2048 26.3 -> 15.5, 768 x 512 x 512 84.5 -> 78.1, 96 x 2048 x 2048 fp16 119.3 -> 116.7; bf16 at that
    // size and beyond stays on the eight-wave 16x16x32 kernel (115.6 against 120.1; 32 x 4096 x 4096 139.9 against
    // 150.6).  Without the softmax they are ahead below two 256-row workgroups per CU (96 x 512 x 512 11.2 -> 10.7,
    // 16 x 512 x 2048 17.0 -> 14.6) and behind from there on (384 x 512 x 512 38.9 against 39.3); where the 64-row
    // workgroups make one and a half rounds of the CUs and the 128-row ones fit in one, the latter stay
    // (48 x 512 x 512 7.5 against 8.2).  B stored [K][L] (its fragments come out of transposing reads): softmax
    // 96 x 512 x 512 13.1 -> 11.8, 12 x 512 x 512 10.0 -> 7.3, 16 x 512 x 2048 26.9 -> 16.6, 768 x 512 x 512
    // 83.8 -> 81.8, level at 96 x 2048 x 2048 (122.7 / 121.6) and 32 x 4096 x 4096 (153.1 / 154.7: stays); without
    // the softmax only the grids that leave CUs empty gain (12 x 512 x 512 7.5 -> 7.0, 8 x 1024 x 1024 10.9 -> 10.0,
    // 16 x 512 x 2048 17.9 -> 16.0; but 96 x 512 x 512 10.7 against 11.6, 48 x 512 x 512 7.5 against 9.0).
    if (plan->d_pad == 64) {
      const bool lk = d->b_layout == DITTO_B_LK;
      const long long n64 = ((d->M + 63) / 64) * d->batch, n128 = ((d->M + 127) / 128) * d->batch;
      bool rows64;
      if (sm)
        rows64 = !((in == DITTO_BF16 || !lk) && n8 >= 2LL * cus && d->L >= 2048);
      else if (lk)
        rows64 = n8 < 2LL * cus && !(n64 > cus && n128 <= cus);
      else
        rows64 = n64 <= cus;
      if (rows64) plan->qt = d->L >= 1024 ? 5 : 4;
      else if (sm && lk && n8 >= 2LL * cus) plan->qt = 6;
    }
    if (d->tile_variant != 0) {
      const int q = d->tile_variant % 10;
      if (d->tile_variant / 10 != plan->d_pad || (q != 1 && q != 2 && q != 4 && q != 5 && q != 8 && q != 9 && q != 6 && q != 7))
        return fail(DITTO_EINVAL, "tile_variant %d cannot run this shape (head_pad %d; q must be 1, 2, 4, 5, 6, 7, 8 or 9)",
                    d->tile_variant, plan->d_pad);
      if ((q == 4 || q == 5) && plan->d_pad != 64)
        return fail(DITTO_EINVAL, "tile_variant %d: the 64-row kernel serves head_pad 64 only", d->tile_variant);
      plan->qt = q;
    }
    const bool kl = d->b_layout == DITTO_B_KL;
    const bool four16 = plan->qt == 4 || plan->qt == 5;  // four waves, 64-row workgroups
    const bool eight = plan->qt >= 6;  // 6, 8, 9: eight waves owning 32 rows each; 7: 48 rows each in some workgroups
    const bool m16 = plan->qt == 6 || plan->qt == 7;
    if (plan->qt == 6 && d->tile_variant == 0 && plan->d_pad == 128) {
      // the planner's own choice between all-256-row blocks (6) and the mix (7)
      if (plan_rows_384(d->M, d->batch, cus) > 0) plan->qt = 7;
    }
    if (plan->qt == 7) {
      plan->nb3 = plan_rows_384(d->M, d->batch, cus);
      if (plan->nb3 == 0 && d->M > 256) plan->nb3 = 1;  // asked for by tile_variant: at least one large block to show for it
    }
    const int bm = four16 ? 64 : eight ? 256 : 128 * plan->qt;
    ditto_tile_param& t = plan->tile;
    t.block_threads = eight ? 512 : 256;
    t.block_m = bm;
    t.block_l = ditto::kBN;
    t.block_n = (int)d->N;
    t.head_pad = plan->d_pad;
    if (four16)
      t.lds_bytes = ditto::bmm_chain4m16_lds_bytes<64>();
    else if (m16)
      t.lds_bytes = plan->d_pad == 64 ? ditto::bmm_chain8m16_lds_bytes<64>() : ditto::bmm_chain8m16_lds_bytes<128>();
    else if (eight)
      t.lds_bytes = plan->d_pad == 64 ? (kl ? ditto::bmm_chain8_lds_bytes<64, true>() : ditto::bmm_chain8_lds_bytes<64, false>())
                                      : (kl ? ditto::bmm_chain8_lds_bytes<128, true>() : ditto::bmm_chain8_lds_bytes<128, false>());
    else
      t.lds_bytes = plan->d_pad == 64 ? ditto::bmm_chain_lds_bytes<64>() : ditto::bmm_chain_lds_bytes<128>();
    plan->nb = (int)((d->M + bm - 1) / bm);
    if (plan->qt == 7) {
      const long long rest = d->M - 384LL * plan->nb3;
      plan->nb = plan->nb3 + (int)(rest > 0 ? (rest + 255) / 256 : 0);
      if (plan->nb3 > 0) t.block_m = 384;  // the larger of the two block sizes
    }
    t.grid_x = (int)(plan->nb * d->batch);
    t.grid_y = t.grid_z = 1;
    t.variant = plan->d_pad * 10 + plan->qt;
    return DITTO_OK;
  }
  if (in == DITTO_F32 || in == DITTO_F64) {
    if (d->acc_dtype != in || d->out_dtype != in)
      return fail(DITTO_EINVAL, "the fp32 / fp64 chain accumulates and outputs its input type");
    if (d->inter_op != DITTO_INTER_CAST && d->inter_op != DITTO_INTER_RELU && d->inter_op != DITTO_INTER_SOFTMAX)
      return fail(DITTO_EUNSUPPORTED, "the fp32 chain takes inter_op cast, relu or softmax");
    if (d->tile_variant != 0) return fail(DITTO_EINVAL, "the fp32 chain has a single variant (tile_variant must be 0)");
    if (d->K > ditto::f32_chain_max_dim() || d->N > ditto::f32_chain_max_dim())
      return fail(DITTO_EUNSUPPORTED, "the fp32 chain supports K, N up to %d", ditto::f32_chain_max_dim());
    if (d->a_row_stride < d->K || d->c_row_stride < d->N || d->f_row_stride < d->N ||
        d->b_row_stride < (d->b_layout == DITTO_B_KL ? d->L : d->K))
      return fail(DITTO_EINVAL, "row stride smaller than row extent");
    if (d->a_row_stride > 0x7fffffff || d->b_row_stride > 0x7fffffff || d->c_row_stride > 0x7fffffff ||
        d->f_row_stride > 0x7fffffff)
      return fail(DITTO_EINVAL, "row stride too large");
    plan->family = 1;
    ditto_tile_param& t = plan->tile;
    t.block_threads = 256;
    t.block_m = 32;
    t.block_n = (int)d->N;
    t.head_pad = 0;
    t.block_l = in == DITTO_F64 ? 32 : 64;
    t.lds_bytes = ditto::f32_chain_lds_bytes_host((int)d->K, (int)d->N, in == DITTO_F64);
    t.grid_x = (int)(((d->M + 31) / 32) * d->batch);
    t.grid_y = t.grid_z = 1;
    t.variant = in == DITTO_F64 ? 1001 : 1000;  // fp32 / fp64 FMA chain
    return DITTO_OK;
  }
  if (in == DITTO_I8) {
    if (d->acc_dtype != DITTO_I32 || (d->out_dtype != DITTO_I32 && d->out_dtype != DITTO_I8))
      return fail(DITTO_EINVAL, "the int8 chain accumulates in int32 and outputs int32 or (the low byte) int8");
    // requantised middle result, or the reference's wrapping cast (optionally behind a ReLU)
    if (d->inter_op != DITTO_INTER_REQUANT && d->inter_op != DITTO_INTER_CAST && d->inter_op != DITTO_INTER_RELU)
      return fail(DITTO_EUNSUPPORTED, "the int8 chain takes inter_op requant, cast (wrapping) or relu (then wrapping)");
    if (d->b_layout != DITTO_B_KL) return fail(DITTO_EUNSUPPORTED, "the int8 chain takes B as [K][L]");
    if (d->K % 16 || d->L % 16 || d->N % 16)
      return fail(DITTO_EINVAL, "K, L and N must be multiples of 16 for the int8 chain");
    if (d->a_row_stride % 16 || d->b_row_stride % 16 || d->c_row_stride % 16 || d->a_batch_stride % 16 ||
        d->b_batch_stride % 16 || d->c_batch_stride % 16)
      return fail(DITTO_EINVAL, "int8 input strides must be multiples of 16 elements");
    if (d->a_row_stride < d->K || d->b_row_stride < d->L || d->c_row_stride < d->N || d->f_row_stride < d->N)
      return fail(DITTO_EINVAL, "row stride smaller than row extent");
    if (d->a_row_stride > 0x7fffffff || d->b_row_stride > 0x7fffffff || d->c_row_stride > 0x7fffffff ||
        d->f_row_stride > 0x7fffffff || d->K > 0x7fffffff / 2 || d->N > 0x7fffffff / 2)
      return fail(DITTO_EINVAL, "extent or row stride too large");
    const long long Lp = (d->L + 255) / 256 * 256;
    if ((d->M + 64) * d->a_row_stride >= 0x7fffffffLL || d->K * d->b_row_stride >= 0x7fffffffLL ||
        Lp * d->c_row_stride >= 0x7fffffffLL)
      return fail(DITTO_EUNSUPPORTED, "a batch entry of A, B or C exceeds 2 GiB");
    // 64-row workgroups halve the weight traffic per row but need twice as many rows to fill the
    // chip; the ring of staged chunks is as deep as LDS allows (four or three stages, else two)
    const int cus = need_device ? device_cus() : 256;
    int mt = ((d->M + 63) / 64) * d->batch >= 2LL * cus ? 2 : 1;
    auto fits = [&](int m, int n) { return ditto::i8_chain_lds_bytes_host((int)Lp, m, n) <= 160 * 1024; };
    int nst = mt == 2 ? 3 : 4;
    if (!fits(mt, nst)) nst = 2;
    if (!fits(mt, nst)) mt = 1, nst = 4;
    if (!fits(mt, nst)) nst = 2;
    if (d->tile_variant != 0) {
      // 8000 + 10 * (row tiles of 32) + ring depth, as select_tile reports it
      const int fm = (d->tile_variant - 8000) / 10, fn = d->tile_variant % 10;
      const bool built = (fm == 1 && (fn == 2 || fn == 4)) || (fm == 2 && (fn == 2 || fn == 3));
      if (d->tile_variant < 8000 || !built || !fits(fm, fn))
        return fail(DITTO_EINVAL, "tile_variant %d cannot run this int8 chain (8012, 8014, 8022 or 8023, within LDS)",
                    d->tile_variant);
      mt = fm, nst = fn;
    }
    const int lds = ditto::i8_chain_lds_bytes_host((int)Lp, mt, nst);
    if (lds > 160 * 1024)
      return fail(DITTO_EUNSUPPORTED, "L=%lld: the requantised row block does not fit in LDS", (long long)d->L);
    plan->family = 2;
    plan->d_pad = mt;
    plan->qt = nst;
    ditto_tile_param& t = plan->tile;
    t.block_threads = ditto::i8_chain_threads();
    t.block_m = 32 * mt;
    t.block_l = (int)Lp;
    t.block_n = 256;
    t.head_pad = 0;
    t.lds_bytes = lds;
    t.grid_x = (int)(((d->M + 32 * mt - 1) / (32 * mt)) * d->batch);
    t.grid_y = t.grid_z = 1;
    t.variant = 8000 + 10 * mt + nst;  // int8 chain: 8000 + 10 * (row tiles of 32) + ring depth
    return DITTO_OK;
  }
  return fail(DITTO_EUNSUPPORTED, "no chain kernel for in_dtype %d", in);
}

struct ConvPlan {
  int px2;             // 0: 1x1 second convolution; 1 | 2: larger one, output-pixel tiles per wave
  size_t w2p_bytes;    // size of the repacked W2 (second part of the workspace, px2 > 0)
  int c1_tiles;
  int ch;              // input channels per staged chunk
  size_t w1p_bytes;    // size of the repacked W1 (the workspace)
  ditto::ConvChainArgs args;
  bool dw;             // depthwise first convolution: dwargs / c2_tiles / dw_shared describe the launch
  int c2_tiles;
  int dw_mode;         // 0 | 1: plain kernel (1: multiplier a multiple of 8); 2 | 3: persistent kernel,
                       // depthwise stage on the matrix cores (2) or the vector ALU (3); 4: the row-streaming
                       // kernel (rowargs); 5: the row-streaming kernel for multiplier 16 (row16args)
  ditto::DwConvArgs dwargs;
  ditto::DwRowsArgs rowargs;
  ditto::Dw16RowsArgs row16args;
  bool resident;       // 1x1 -> 3x3 with at most 64 channels: persistent kernel, W2 resident in LDS
  int res_grid;
  ditto::ConvResidentArgs rargs;
  bool rows13;         // 1x1 -> 3x3 with at most 64 channels everywhere: the same pipeline (cvargs.f13), W2 fragments
                       // in the workspace
  bool rows31;         // 3x3 -> 1x1 with at most 64 -> 64 -> 256 channels: the row pipeline (cvargs), W1 fragments
                       // in the workspace
  ditto::ConvRowsArgs cvargs;
  ditto_tile_param tile;
};

// Depthwise first convolution + 1x1 second (dw_conv_chain.h): everything in one kernel, no workspace.
// dw_mode 2 | 3: the persistent kernel, depthwise stage on the matrix cores (multipliers that are
// multiples of 16) or on the vector ALU (3x3, multiplier 1, 2, 4, 8); dw_mode 0 | 1: the plain
// kernel for what is left (1: multiples of 8, 0: 1, 2, 4).
// dw_mode 4: the row-streaming kernel (dw_rows.h) for multiplier 1, 3x3, pad 1, stride 1, at most 32 input and
// 64 output channels, image rows of whole 16-byte vectors and at most 128 pixels, 16-bit output.
// vec_cap: the widest halo vector (elements) the pointer of this call allows; 8 when planning without one.
// DITTO_DW_ROWS=0 keeps such shapes on the persistent kernel (A/B runs, tests of that kernel).
// dw_mode 5: the row-streaming kernel for multiplier 16 (dw16_rows.h): 3x3, pad 1, stride 1, an even number of at
// most 32 input channels, at most 64 output channels, image rows of whole 16-byte vectors whose ring of row slots
// fits beside the filters in LDS, 16-bit output.  DITTO_DW16_ROWS=0 keeps such shapes on the persistent kernel.
// What a forced tile_variant allows (0: everything; see ditto_conv_chain_desc.tile_variant).
struct ConvSteer {
  int tv = 0;
  bool rows = true;      // 3700 / 3800: the row pipelines
  bool resident = true;  // 3600: the persistent kernel with W2 resident in LDS
  bool dw_rows = true;   // 4024
  bool dw16_rows = true; // 4025
  bool persist = false;  // 3900: the persistent 3x3 -> 1x1 kernel (switched off)
};
int conv_steer(int tv, ConvSteer* st) {
  *st = ConvSteer();
  st->tv = tv;
  if (tv == 0) return DITTO_OK;
  if (tv < 0) return fail(DITTO_EINVAL, "tile_variant must be 0, a variant id or a family id");
  const int fam = tv / 100 * 100;
  st->rows = fam == 3700 || fam == 3800;
  st->resident = fam == 3600;
  st->dw_rows = tv == 4024;
  st->dw16_rows = tv == 4025;
  st->persist = fam == 3900;
  if (!(fam == 3000 || fam == 3100 || fam == 3500 || fam == 3600 || fam == 3700 || fam == 3800 || fam == 3900 || fam == 4000))
    return fail(DITTO_EINVAL, "tile_variant %d names no conv chain kernel family", tv);
  return DITTO_OK;
}
// The plan that came out against the variant that was asked for: a family id (a multiple of 100; 3000 also stands
// for the 16-channel-chunk form 31xx, 4000 for every depthwise kernel but the two row-streaming ones) or an exact id.
int conv_steer_check(const ConvSteer& st, int got) {
  if (st.tv == 0 || st.tv == got) return DITTO_OK;
  if (st.tv % 100 == 0) {
    const int fam = got / 100 * 100;
    if (fam == st.tv || (st.tv == 3000 && fam == 3100)) {
      if (st.tv != 4000 || (got != 4024 && got != 4025)) return DITTO_OK;
    }
  }
  return fail(DITTO_EINVAL, "tile_variant %d cannot run this chain (the kernel that fits it under that constraint is %d)",
              st.tv, got);
}

int plan_dw_conv(const ditto_conv_chain_desc* d, const ConvSteer& steer, long long P, long long Q, ConvPlan* plan,
                 bool need_device, bool allow_dwv = true, int vec_cap = 8, bool allow_rows = true) {
  if (d->C1 % d->C0) return fail(DITTO_EINVAL, "depthwise: C1 must be a multiple of C0");
  const long long mult = d->C1 / d->C0;
  const long long RS = d->R1 * d->S1;
  if (!(d->R2 == 1 && d->S2 == 1 && d->pad2 == 0 && d->stride2 == 1))
    return fail(DITTO_EUNSUPPORTED, "depthwise chain: the second convolution must be 1x1, stride 1, no padding");
  // the persistent kernel: depthwise stage on the matrix cores (multipliers that are multiples of 16)
  // or, for 3x3 filters with multiplier 1, 2, 4, 8 (and whole 16-byte vectors of W1, W2), on the vector ALU
  // (that variant is built with the 16-byte output stores only: output rows of a multiple of 8, not fp32)
  const bool dwv = allow_dwv && d->R1 == 3 && d->S1 == 3 && (mult == 1 || mult == 2 || mult == 4 || mult == 8) &&
                   d->C1 % 8 == 0 && Q % 8 == 0 && d->out_dtype != DITTO_F32;
  const bool mfma = (mult % 16 == 0 && RS <= ditto::kDwMfmaTaps) || dwv;
  if (!mfma && RS > 2 * ditto::kDwPairs - 1)
    return fail(DITTO_EUNSUPPORTED,
                "depthwise chain: filters of at most 9 taps (16 when the channel multiplier is a multiple of 16)");
  if (!(mult == 1 || mult == 2 || mult == 4 || mult % 8 == 0))
    return fail(DITTO_EUNSUPPORTED, "depthwise chain: channel multiplier must be 1, 2, 4 or a multiple of 8");
  if (d->C2 > 256) return fail(DITTO_EUNSUPPORTED, "depthwise chain: at most 256 output channels");
  if (d->C1 > 32768) return fail(DITTO_EUNSUPPORTED, "depthwise chain: at most 32768 intermediate channels");
  memset(plan, 0, sizeof(*plan));
  plan->dw = true;
  if (allow_rows && vec_cap >= 8 && steer.dw_rows && mult == 1 && d->R1 == 3 && d->S1 == 3 && d->pad1 == 1 &&
      d->stride1 == 1 && d->C0 <= ditto::kDwRowsC && d->C2 <= 64 && d->W % 8 == 0 && d->W <= 128 &&
      d->out_dtype != DITTO_F32 && d->H * d->W * 64 < 0x7fffffffLL) {
    // Bands of whole output rows, one workgroup each: all input rows of a band stay in LDS.  Among the
    // band heights that fit, the one with the fewest row steps on the busiest CU (a band costs its rows
    // plus the two halo rows plus about three steps of start-up).
    const int cus = need_device ? device_cus() : 256;
    int band_max = 0;
    while (band_max < d->H && ditto::dw_rows_lds_bytes((int)d->W, band_max + 1) <= 160 * 1024) ++band_max;
    if (band_max >= 1) {
      long long best = -1;
      int best_nb = 0;
      const int nb_min = (int)((d->H + band_max - 1) / band_max);
      for (int nb = nb_min; nb <= d->H && nb < nb_min + 64; ++nb) {
        const int band = (int)((d->H + nb - 1) / nb);
        const long long wgs = d->N * ((d->H + band - 1) / band);
        const long long cost = ((wgs + cus - 1) / cus) * (band + 5);
        if (best < 0 || cost < best) { best = cost; best_nb = nb; }
      }
      ditto::DwRowsArgs& r = plan->rowargs;
      r.N = (int)d->N; r.C0 = (int)d->C0; r.H = (int)d->H; r.W = (int)d->W; r.C2 = (int)d->C2;
      r.band = (int)((d->H + best_nb - 1) / best_nb);
      r.bands = (int)((d->H + r.band - 1) / r.band);
      r.relu_mid = d->inter_op == DITTO_INTER_RELU;
      r.relu_out = d->relu_out != 0;
      plan->dw_mode = 4;
      plan->c2_tiles = 2;
      ditto_tile_param& t = plan->tile;
      t.block_threads = 64 * ditto::kDwRowsWaves;
      t.block_m = r.band * r.W;
      t.block_l = ditto::kDwRowsC;
      t.block_n = 64;
      t.head_pad = 0;
      t.lds_bytes = ditto::dw_rows_lds_bytes(r.W, r.band);
      t.grid_x = r.N * r.bands;
      t.grid_y = r.band;
      t.grid_z = r.W;
      t.variant = 4000 + 20 + 4;
      return DITTO_OK;
    }
  }
  if (allow_rows && vec_cap >= 8 && steer.dw16_rows && mult == 16 && d->R1 == 3 && d->S1 == 3 && d->pad1 == 1 &&
      d->stride1 == 1 && d->C0 <= 32 && d->C0 % 2 == 0 && d->C2 <= 64 && d->W % 8 == 0 && d->W >= 8 &&
      ditto::dw16_rows_ni((int)d->C0, (int)d->W) <= 8 &&
      ditto::dw16_rows_lds_bytes((int)d->C0, (int)d->W) <= 160 * 1024 && d->out_dtype != DITTO_F32 &&
      d->H * d->W < (1 << 20)) {
    // Bands of whole output rows, one workgroup each, whose pixels eight waves take as one stream of 32-pixel
    // tiles: the band height with the fewest tiles on the busiest SIMD (waves w and w + 4 share one) over
    // the rounds of workgroups, a workgroup's start-up counted as three tiles.
    const int cus = need_device ? device_cus() : 256;
    long long best = -1;
    int best_band = 1;
    for (int nb = 1; nb <= d->H; ++nb) {
      const int band = (int)((d->H + nb - 1) / nb);
      if (nb > 1 && band == (int)((d->H + nb - 2) / (nb - 1))) continue;
      const long long wgs = d->N * ((d->H + band - 1) / band);
      const long long ntiles = (band * d->W + 31) / 32;
      const long long q = ntiles / ditto::kDw16Compute, rem = ntiles % ditto::kDw16Compute;
      const long long busiest = 2 * q + (rem > 0) + (rem > 4);
      const long long cost = ((wgs + cus - 1) / cus) * (busiest + 3);
      if (best < 0 || cost <= best) { best = cost; best_band = band; }
    }
    ditto::Dw16RowsArgs& r = plan->row16args;
    r.N = (int)d->N; r.C0 = (int)d->C0; r.H = (int)d->H; r.W = (int)d->W; r.C2 = (int)d->C2;
    r.band = best_band;
    r.bands = (int)((d->H + r.band - 1) / r.band);
    r.ring = ditto::dw16_rows_ring(r.W);
    r.relu_mid = d->inter_op == DITTO_INTER_RELU;
    r.relu_out = d->relu_out != 0;
    plan->dw_mode = 5;
    plan->c2_tiles = 2;
    ditto_tile_param& t = plan->tile;
    t.block_threads = 64 * ditto::kDw16Waves;
    t.block_m = r.band * r.W;
    t.block_l = (int)d->C1;
    t.block_n = 64;
    t.head_pad = 0;
    t.lds_bytes = ditto::dw16_rows_lds_bytes(r.C0, r.W);
    t.grid_x = r.N * r.bands;
    t.grid_y = r.band;
    t.grid_z = r.W;
    t.variant = 4000 + 20 + 5;
    return DITTO_OK;
  }
  plan->dw_mode = dwv ? 3 : mfma ? 2 : mult % 8 == 0 ? 1 : 0;
  const int c2t = d->C2 <= 32 ? 1 : d->C2 <= 64 ? 2 : d->C2 <= 128 ? 4 : 8;
  const int pxw = mfma ? ditto::dw_mfma_pxw(c2t) : c2t == 8 ? 1 : 2;
  const int groups = mfma ? ditto::dw_mfma_groups(c2t) : 1;
  const int slots = 128 * groups * pxw;  // pixels of a workgroup's tile
  ditto::DwConvArgs& a = plan->dwargs;
  a.N = (int)d->N; a.C0 = (int)d->C0; a.H = (int)d->H; a.W = (int)d->W;
  a.mult = (int)mult; a.C1 = (int)d->C1; a.R = (int)d->R1; a.S = (int)d->S1;
  a.pad = (int)d->pad1; a.stride = (int)d->stride1; a.C2 = (int)d->C2; a.P = (int)P; a.Q = (int)Q;
  // Pixel tile: the split of the output plane into TH x TW pieces of at most `slots` pixels that
  // costs the fewest 32-pixel tile rounds (a round = one tile on each wave; the plain kernel always
  // runs all its rounds); ties go to the wider tile.  Where 16-byte output stores are possible only
  // tile widths that keep them (multiples of 8) are considered.
  const bool want_wide = mfma && d->out_dtype != DITTO_F32 && Q % 8 == 0;
  for (int pass = want_wide ? 0 : 1; pass < 2; ++pass) {  // pass 0: only widths that are multiples of 8
    long long best = -1;
    for (int k = 1; k <= (int)Q; ++k) {
      const int tw = (int)((Q + k - 1) / k);
      if (tw > slots) continue;
      if (tw < 8 && k > 1) break;
      if (pass == 0 && tw % 8) continue;
      int th = slots / tw;
      if (th > P) th = (int)P;
      const long long th_n = (P + th - 1) / th;
      th = (int)((P + th_n - 1) / th_n);
      const long long tw_n = (Q + tw - 1) / tw;
      const long long rounds = mfma ? ((th * tw + 31) / 32 + 4 * groups - 1) / (4 * groups) : pxw;
      const long long cost = th_n * tw_n * rounds;
      if (best < 0 || cost < best) { best = cost; a.TH = th; a.TW = tw; }
    }
    if (best >= 0) break;
  }
  // input channels per chunk: chx * mult a multiple of the MFMA block (32 intermediate channels
  // on the matrix-core path, 16 on the vector path); as many channels as keep two workgroups on a
  // CU, else as many as fit at all, else a smaller pixel tile
  const int cm_unit = mfma ? 32 : 16;
  int step = 1;
  while ((step * mult) % cm_unit) ++step;
  // halo loads: vectors of up to 8 elements that divide W (the run call narrows them if x is less
  // aligned); output through 16-byte stores when rows allow
  const int vec_max = mfma ? (d->W % 8 == 0 && vec_cap >= 8 ? 8 : d->W % 4 == 0 ? 4 : d->W % 2 == 0 ? 2 : 1) : 1;
  a.vec = vec_max;
  a.wide = mfma && d->out_dtype != DITTO_F32 && Q % 8 == 0 && a.TW % 8 == 0;
  auto lds_of = [&](int chx) {
    return mfma ? ditto::dw_conv_mfma_lds_bytes(chx, a.mult, a.rows_in, a.cols_al, 32 * c2t, groups, a.wide != 0)
                : ditto::dw_conv_lds_bytes(chx, a.mult, a.rows_in, a.cols_in, 32 * c2t) + 16;
  };
  // the MFMA kernel keeps a chunk's halo tile in flight in registers (kDwXpf vectors per thread)
  // and addresses it with packed 32-bit offsets
  auto fits_regs = [&](int chx) {
    if (!mfma) return true;
    // a thread owns one (row, vector) position of the halo tile and walks the channels, `cphases`
    // at a time: kDwXpf passes must cover the chunk
    const int nvr = a.cols_al / a.vec;
    const int cphases = (256 * groups / nvr) / a.rows_in;
    const int passes_max = a.vec == 8 ? ditto::kDwXpf / 2 : ditto::kDwXpf;  // a 16-byte vector takes two entries
    return cphases >= 1 && (chx + cphases - 1) / cphases <= passes_max &&
           (long long)(chx + 1) * d->H * d->W < 0x7fffffffLL;
  };
  const int chx_max = (int)((d->C0 + step - 1) / step) * step;
  int lds = 0;
  for (;;) {
    a.rows_in = (a.TH - 1) * a.stride + a.R;
    a.cols_in = (a.TW - 1) * a.stride + a.S;
    a.chx = 0;
    // everything resident (one chunk, filters staged once per workgroup) with the widest loads
    // that leave room for it ...
    for (int vec = vec_max; mfma && vec >= 1 && !a.chx; vec >>= 1) {
      a.vec = vec;
      a.cols_al = (a.cols_in + 2 * vec - 2) / vec * vec;
      a.cols_al += a.cols_al & 1;
      // 16-byte vectors halve the load and LDS-write instructions of the halo staging (5-6 % of the
      // kernel on 16-wide tiles) but pad the halo rows more: not where that is over a third
      if (vec == 8 && 3 * a.cols_al > 4 * ((a.cols_in + 6) / 4 * 4)) continue;
      lds = lds_of(chx_max);
      if (lds <= 160 * 1024 && fits_regs(chx_max)) a.chx = chx_max;
    }
    // ... else chunks: small enough for two workgroups per CU, else whatever fits
    if (!a.chx) {
      a.vec = vec_max;  // 16-byte vectors under the same padding rule as above
      if (a.vec == 8 && 3 * ((a.cols_in + 14) / 8 * 8) > 4 * ((a.cols_in + 6) / 4 * 4)) a.vec = 4;
      a.cols_al = (a.cols_in + 2 * a.vec - 2) / a.vec * a.vec;
      a.cols_al += a.cols_al & 1;
      for (int limit : {78 * 1024, 150 * 1024}) {
        for (int chx = chx_max; chx >= step; chx -= step) {
          lds = lds_of(chx);
          if (lds <= limit && fits_regs(chx)) { a.chx = chx; break; }
        }
        if (a.chx) break;
      }
    }
    if (a.chx) break;
    if (a.TH > 1) a.TH = (a.TH + 1) / 2;
    else if (a.TW > 16) { a.TW = (a.TW + 1) / 2; a.wide = a.wide && a.TW % 8 == 0; }
    else return fail(DITTO_EUNSUPPORTED, "depthwise chain tile does not fit in LDS");
  }
  {  // same number of chunks, evenly sized
    const int chunks = (int)((d->C0 + a.chx - 1) / a.chx);
    const int even = (int)((d->C0 + chunks - 1) / chunks);
    a.chx = (even + step - 1) / step * step;
    lds = lds_of(a.chx);
  }
  a.tiles_h = (int)((P + a.TH - 1) / a.TH);
  a.tiles_w = (int)((Q + a.TW - 1) / a.TW);
  a.relu_mid = d->inter_op == DITTO_INTER_RELU;
  a.relu_out = d->relu_out != 0;
  a.out_f32 = d->out_dtype == DITTO_F32;
  if (dwv && !a.wide) return plan_dw_conv(d, steer, P, Q, plan, need_device, false, vec_cap, false);  // that variant needs the wide stores
  plan->c2_tiles = c2t;
  ditto_tile_param& t = plan->tile;
  t.block_threads = 256 * groups;
  t.block_m = a.TH * a.TW;
  t.block_l = a.chx * a.mult;
  t.block_n = 32 * c2t;
  t.head_pad = 0;
  t.lds_bytes = lds;
  t.grid_x = a.N * a.tiles_h * a.tiles_w;
  if (mfma) {  // persistent workgroups, as many as the CUs hold at this LDS footprint
    // two workgroups per CU where LDS and registers allow: the eight-wave variants use more than
    // 128 registers per lane, so only one of them fits
    const int per_cu = (groups == 1 && 160 * 1024 / lds >= 2) ? 2 : 1;
    const int cap = (need_device ? device_cus() : 256) * per_cu;
    if (t.grid_x > cap) t.grid_x = cap;
    a.grid = t.grid_x;
    a.nt_store = (a.TW * 2) % 128 == 0;
  }
  t.grid_y = a.TH;
  t.grid_z = a.TW;
  t.variant = 4000 + c2t * 10 + plan->dw_mode;
  return DITTO_OK;
}

int plan_conv_steered(const ditto_conv_chain_desc* d, const ConvSteer& steer, ConvPlan* plan, bool need_device,
                      int dw_vec_cap, bool allow_resident, bool allow_dw_rows);

// allow_resident = false: the general kernels only (pointers the specialised ones cannot take);
// allow_dw_rows: y takes 16-byte stores
int plan_conv(const ditto_conv_chain_desc* d, ConvPlan* plan, bool need_device = false, int dw_vec_cap = 8,
              bool allow_resident = true, bool allow_dw_rows = true) {
  if (!d) return fail(DITTO_EINVAL, "null descriptor");
  ConvSteer steer;
  int rc = conv_steer(d->tile_variant, &steer);
  if (rc != DITTO_OK) return rc;
  rc = plan_conv_steered(d, steer, plan, need_device, dw_vec_cap, allow_resident, allow_dw_rows);
  if (rc != DITTO_OK) return rc;
  return conv_steer_check(steer, plan->tile.variant);
}

int plan_conv_steered(const ditto_conv_chain_desc* d, const ConvSteer& steer, ConvPlan* plan, bool need_device,
                      int dw_vec_cap, bool allow_resident, bool allow_dw_rows) {
  if (d->abi_version != DITTO_CHAIN_ABI_VERSION)
    return fail(DITTO_EINVAL, "descriptor abi_version %d, library %d", d->abi_version, DITTO_CHAIN_ABI_VERSION);
  if (d->in_dtype != DITTO_F16 && d->in_dtype != DITTO_BF16)
    return fail(DITTO_EUNSUPPORTED, "conv chains are built for fp16 / bf16 (in_dtype %d)", d->in_dtype);
  if (d->acc_dtype != DITTO_F32) return fail(DITTO_EUNSUPPORTED, "conv chains accumulate in fp32");
  if (d->out_dtype != d->in_dtype && d->out_dtype != DITTO_F32)
    return fail(DITTO_EINVAL, "out_dtype must be in_dtype or fp32");
  if (d->inter_op != DITTO_INTER_CAST && d->inter_op != DITTO_INTER_RELU)
    return fail(DITTO_EINVAL, "inter_op %d not valid for a conv chain", d->inter_op);
  if (d->N <= 0 || d->C0 <= 0 || d->H <= 0 || d->W <= 0 || d->C1 <= 0 || d->C2 <= 0 || d->R1 <= 0 ||
      d->S1 <= 0 || d->R2 <= 0 || d->S2 <= 0 || d->stride1 <= 0 || d->stride2 <= 0 || d->pad1 < 0 || d->pad2 < 0)
    return fail(DITTO_EINVAL, "conv extents must be positive and paddings non-negative");
  const bool dw = d->groups1 != 0 && d->groups1 != 1;
  if (dw && d->groups1 != d->C0) return fail(DITTO_EUNSUPPORTED, "groups1 must be 1 (dense) or C0 (depthwise)");
  const bool second_1x1 = d->R2 == 1 && d->S2 == 1 && d->pad2 == 0;
  // A strided 1x1 second convolution keeps every stride2-th pixel of the intermediate image and nothing else: the
  // chain is the same chain with the first convolution strided by stride1 * stride2 (output p of the second reads
  // intermediate p * stride2, i.e. input rows from p * stride1 * stride2 - pad1 on; the number of outputs agrees,
  // floor(floor(x / s1) / s2) = floor(x / (s1 s2))).  Planned and run that way.
  ditto_conv_chain_desc folded;
  if (second_1x1 && d->stride2 > 1) {
    if (d->stride1 * d->stride2 > 0x7fff) return fail(DITTO_EINVAL, "strides too large");
    folded = *d;
    folded.stride1 = d->stride1 * d->stride2;
    folded.stride2 = 1;
    d = &folded;
  }
  if (dw && d->stride2 != 1) return fail(DITTO_EUNSUPPORTED, "depthwise chain: the second convolution must be 1x1");
  if (!dw) {
    if (!second_1x1 && (d->R2 > 3 || d->S2 > 3))
      return fail(DITTO_EUNSUPPORTED, "a second convolution larger than 1x1 takes filters up to 3x3");
    if (!second_1x1 && d->stride2 > 4) return fail(DITTO_EUNSUPPORTED, "second convolution: strides up to 4");
    if (d->C1 % 8) return fail(DITTO_EINVAL, "C1 must be a multiple of 8");
    if (d->C1 > 256) return fail(DITTO_EUNSUPPORTED, "C1=%lld: at most 256 intermediate channels", (long long)d->C1);
  }
  if (d->R1 > 7 || d->S1 > 7) return fail(DITTO_EUNSUPPORTED, "first filter larger than 7x7");
  const long long P = (d->H + 2 * d->pad1 - d->R1) / d->stride1 + 1;
  const long long Q = (d->W + 2 * d->pad1 - d->S1) / d->stride1 + 1;
  if (d->H + 2 * d->pad1 < d->R1 || d->W + 2 * d->pad1 < d->S1 || P <= 0 || Q <= 0)
    return fail(DITTO_EINVAL, "empty convolution output");
  if (d->N * d->C0 * d->H * d->W > 0x7fffffffLL * 4 || d->N * d->C2 * P * Q > 0x7fffffffLL * 4 ||
      d->H > 65535 || d->W > 65535 || d->N > 65535 || d->C0 > 65535 || d->C2 > 65535)
    return fail(DITTO_EINVAL, "tensor too large");
  // (a y that is not 16-byte aligned rules out both kernels that only store 16-byte vectors)
  if (dw) return plan_dw_conv(d, steer, P, Q, plan, need_device, allow_dw_rows, dw_vec_cap, allow_dw_rows);
  memset(plan, 0, sizeof(*plan));
  const int c1t = d->C1 <= 32 ? 1 : d->C1 <= 64 ? 2 : d->C1 <= 128 ? 4 : 8;
  const int pxw = c1t == 8 ? 1 : 2;
  const int slots = 128 * pxw;
  ditto::ConvChainArgs& a = plan->args;
  a.N = (int)d->N; a.C0 = (int)d->C0; a.H = (int)d->H; a.W = (int)d->W;
  a.C1 = (int)d->C1; a.R = (int)d->R1; a.S = (int)d->S1; a.pad = (int)d->pad1; a.stride = (int)d->stride1;
  a.C2 = (int)d->C2; a.P = (int)P; a.Q = (int)Q;
  if (!second_1x1) {
    // The first convolution produces the output tile grown by the second filter's halo (recomputed
    // per workgroup) into at most `slots` pixel slots; the second reads it from LDS.
    const int s2 = (int)d->stride2;
    if (P + 2 * d->pad2 < d->R2 || Q + 2 * d->pad2 < d->S2) return fail(DITTO_EINVAL, "empty convolution output");
    const long long P2 = (P + 2 * d->pad2 - d->R2) / s2 + 1, Q2 = (Q + 2 * d->pad2 - d->S2) / s2 + 1;
    if (P2 <= 0 || Q2 <= 0) return fail(DITTO_EINVAL, "empty convolution output");
    if (d->N * d->C2 * P2 * Q2 > 0x7fffffffLL * 4) return fail(DITTO_EINVAL, "tensor too large");
    a.R2 = (int)d->R2; a.S2 = (int)d->S2; a.pad2 = (int)d->pad2; a.P2 = (int)P2; a.Q2 = (int)Q2;
    a.stride2 = s2;
    // 1x1 -> 3x3 (pad 1) with at most 64 channels everywhere, 16-bit output and image rows of whole 16-byte
    // vectors up to 64 pixels: the row pipeline with the 1x1 convolution in its transposing stage (conv_rows.h)
    if (allow_resident && steer.rows && s2 == 1 && d->R1 == 1 && d->S1 == 1 && d->pad1 == 0 &&
        d->stride1 == 1 && d->R2 == 3 && d->S2 == 3 && d->pad2 == 1 && d->C0 <= ditto::kCvrC && d->C1 <= ditto::kCvrC &&
        d->C2 <= ditto::kCvrC && d->C0 % 8 == 0 && d->W % 8 == 0 && d->W <= 64 && d->out_dtype != DITTO_F32 &&
        d->C0 * d->H * d->W * 2 < 0x7fffffffLL) {
      const int cus = need_device ? device_cus() : 256;
      int band_max = ditto::conv_rows_band_max((int)d->W);
      if (band_max > d->H) band_max = (int)d->H;
      while (band_max >= 1 && ditto::conv_rows_lds_bytes((int)d->W, band_max, true) > 160 * 1024) --band_max;
      if (band_max >= 1) {
        // fewest steps of two rows on the busiest CU (a band costs its steps plus about three of start-up)
        long long best = -1;
        int best_nb = 0;
        const int nb_min = (int)((d->H + band_max - 1) / band_max);
        for (int nb = nb_min; nb <= d->H && nb < nb_min + 64; ++nb) {
          const int band = (int)((d->H + nb - 1) / nb);
          const long long wgs = d->N * ((d->H + band - 1) / band);
          const long long cost = ((wgs + cus - 1) / cus) * ((band + 1) / 2 + 3);
          if (best < 0 || cost <= best) { best = cost; best_nb = nb; }  // ties: the split that fills more CUs
        }
        ditto::ConvRowsArgs& r = plan->cvargs;
        r.N = (int)d->N; r.C0 = (int)d->C0; r.H = (int)d->H; r.W = (int)d->W;
        r.Cm = (int)d->C1; r.C1 = (int)d->C2; r.C2 = (int)d->C2;
        r.band = (int)((d->H + best_nb - 1) / best_nb);
        r.bands = (int)((d->H + r.band - 1) / r.band);
        r.f13 = 1;
        r.relu_pre = d->inter_op == DITTO_INTER_RELU;
        r.relu_mid = d->relu_out != 0;
        r.relu_out = 0;
        plan->rows13 = true;
        plan->c1_tiles = 2;
        plan->px2 = 1;
        plan->w1p_bytes = 0;
        plan->w2p_bytes = ditto::kCvrW1Bytes;
        ditto_tile_param& t = plan->tile;
        t.block_threads = 64 * ditto::kCvrWaves;
        t.block_m = r.band * r.W;
        t.block_l = ditto::kCvrC;
        t.block_n = (int)d->C2;
        t.head_pad = ditto::kCvrC;
        t.lds_bytes = ditto::conv_rows_lds_bytes(r.W, r.band, true);
        t.grid_x = r.N * r.bands;
        t.grid_y = r.band;
        t.grid_z = r.W;
        t.variant = 3800 + r.band;  // row pipeline, 1x1 first; output rows per workgroup
        return DITTO_OK;
      }
    }
    // 1x1 -> 3x3 (pad 1) with at most 64 channels everywhere and rows that are whole 16-byte vectors: the
    // persistent kernel that keeps W2 in LDS (conv_chain_resident.h), tiles of whole output rows
    if (allow_resident && steer.resident && s2 == 1 && d->R1 == 1 && d->S1 == 1 && d->pad1 == 0 && d->stride1 == 1 && d->R2 == 3 &&
        d->S2 == 3 && d->pad2 == 1 && d->C0 <= ditto::kCrC && d->C1 <= ditto::kCrC && d->C2 <= ditto::kCrC &&
        d->C0 % 8 == 0 && d->W % 8 == 0 && d->W <= 256 &&
        d->C0 * d->H * d->W * 2 < 0x7fffffffLL) {
      int th2 = (int)(256 / d->W);
      if (th2 > d->H) th2 = (int)d->H;
      while (th2 >= 1 && (ditto::conv_resident_lds_bytes(th2, (int)d->W) > 160 * 1024 ||
                          (th2 + 2) * d->W > 64 * ditto::kCrMaxLoads))
        --th2;
      if (th2 >= 1) {
        const int cus = need_device ? device_cus() : 256;
        ditto::ConvResidentArgs& r = plan->rargs;
        r.N = (int)d->N; r.C0 = (int)d->C0; r.H = (int)d->H; r.W = (int)d->W; r.C1 = (int)d->C1; r.C2 = (int)d->C2;
        r.TH2 = th2;
        r.tiles_h = (int)((d->H + th2 - 1) / th2);
        r.ntiles = r.N * r.tiles_h;
        r.relu_mid = d->inter_op == DITTO_INTER_RELU;
        r.relu_out = d->relu_out != 0;
        r.out_f32 = d->out_dtype == DITTO_F32;
        plan->resident = true;
        plan->res_grid = r.ntiles < cus ? r.ntiles : cus;
        plan->px2 = 1;
        plan->w1p_bytes = 0;
        plan->w2p_bytes = ditto::kCrW2Bytes;
        ditto_tile_param& t = plan->tile;
        t.block_threads = 512;
        t.block_m = th2 * (int)d->W;
        t.block_l = ditto::kCrC;
        t.block_n = (int)d->C2;
        t.head_pad = ditto::kCrC;
        t.lds_bytes = ditto::conv_resident_lds_bytes(th2, (int)d->W);
        t.grid_x = plan->res_grid;
        t.grid_y = th2;
        t.grid_z = (int)d->W;
        t.variant = 3600 + th2;  // persistent, W2 resident in LDS; th2 output rows per tile
        return DITTO_OK;
      }
    }
    // an output tile of TH2 x TW2 pixels needs the intermediate pixels (TH2 - 1) s2 + R2 by (TW2 - 1) s2 + S2
    a.TW2 = (int)Q2;
    while (((a.TW2 - 1) * s2 + a.S2) * a.R2 > slots) a.TW2 = (a.TW2 + 1) / 2;
    a.TW = (a.TW2 - 1) * s2 + a.S2;
    a.TH = slots / a.TW;
    if (a.TH > (P2 - 1) * s2 + a.R2) a.TH = (int)(P2 - 1) * s2 + a.R2;
    a.TH2 = (a.TH - a.R2) / s2 + 1;
    a.TH = (a.TH2 - 1) * s2 + a.R2;
    a.rows_in = (a.TH - 1) * a.stride + a.R;
    a.cols_in = (a.TW - 1) * a.stride + a.S;
    const int RS1 = a.R * a.S;
    int lds = ditto::conv_chain_lds_bytes(a.rows_in, a.cols_in, RS1, 32 * c1t, 32);
    a.wide2 = d->out_dtype != DITTO_F32 && Q2 % 8 == 0 && a.TW2 % 8 == 0;
    const int lds2 = ditto::conv_chain2_lds_bytes(slots, 32 * c1t, a.S2, a.wide2 != 0);
    if (lds2 > lds) lds = lds2;
    if (lds > 160 * 1024) return fail(DITTO_EUNSUPPORTED, "conv chain tile does not fit in LDS");
    a.tiles_h = (int)((P2 + a.TH2 - 1) / a.TH2);
    a.tiles_w = (int)((Q2 + a.TW2 - 1) / a.TW2);
    a.relu_mid = d->inter_op == DITTO_INTER_RELU;
    a.relu_out = d->relu_out != 0;
    a.out_f32 = d->out_dtype == DITTO_F32;
    plan->c1_tiles = c1t;
    plan->ch = 32;
    plan->px2 = a.TH2 * a.TW2 <= 128 ? 1 : 2;
    plan->w1p_bytes = ((size_t)ditto::conv_w1_chunk_bytes(RS1, 32 * c1t, 32) * (size_t)((d->C0 + 31) / 32) + 255) / 256 * 256;
    plan->w2p_bytes = (size_t)ditto::conv_w2_chunk_bytes(a.R2 * a.S2) * (size_t)((d->C2 + 63) / 64) * (size_t)c1t;
    ditto_tile_param& t = plan->tile;
    t.block_threads = 256;
    t.block_m = a.TH2 * a.TW2;
    t.block_l = 32 * c1t;
    t.block_n = (int)d->C2;
    t.head_pad = 32;
    t.lds_bytes = lds;
    t.grid_x = a.N * a.tiles_h * a.tiles_w;
    t.grid_y = a.TH2;
    t.grid_z = a.TW2;
    t.variant = 3500 + c1t * 10 + plan->px2;  // second convolution through LDS
    return DITTO_OK;
  }
  // 3x3 (pad 1, stride 1) -> 1x1 with at most 64 input and intermediate and 256 output channels, image rows of
  // whole 16-byte vectors up to 64 pixels, 16-bit output: the row pipeline (conv_rows.h).  Bands of whole
  // output rows, one workgroup each; a band's rows are all in flight at once, which bounds its height.
  if (allow_resident && steer.rows && !steer.persist && d->R1 == 3 && d->S1 == 3 && d->pad1 == 1 &&
      d->stride1 == 1 && d->C0 <= ditto::kCvrC && d->C1 <= ditto::kCvrC && d->C2 <= 256 && d->W % 8 == 0 && d->W <= 64 &&
      d->out_dtype != DITTO_F32 && d->C0 * d->H * d->W * 2 < 0x7fffffffLL && d->C2 * d->H * d->W * 2 < 0x7fffffffLL &&
      // where it pays (measured against the general kernel): the pipeline pads C0 and C1 to 64, and its gain is the
      // output stream under the compute - wide outputs - or, with few images, more workgroups than the general
      // kernel's tiles of 256 pixels (32 x 32 x 56 x 56 -> 32 -> 128: 16.4 against 12.3 us; 64 -> 64 -> 64: a tie;
      // one image 64 -> 64 -> 256: 8.9 against 15.6 us)
      (steer.tv / 100 == 37 ||
       ((d->C0 > 32 || d->C1 > 32) &&
      (d->C2 >= 192 || d->N * ((P + (256 / d->W > 0 ? 256 / d->W : 1) - 1) / (256 / d->W > 0 ? 256 / d->W : 1)) <
                           (need_device ? device_cus() : 256))))) {
    const int cus = need_device ? device_cus() : 256;
    int band_max = ditto::conv_rows_band_max((int)d->W);
    if (band_max > d->H) band_max = (int)d->H;
    while (band_max >= 1 && ditto::conv_rows_lds_bytes((int)d->W, band_max) > 160 * 1024) --band_max;
    if (band_max >= 1) {
      // fewest steps of two rows on the busiest CU (a band costs its steps plus about three of start-up)
      long long best = -1;
      int best_nb = 0;
      const int nb_min = (int)((d->H + band_max - 1) / band_max);
      for (int nb = nb_min; nb <= d->H && nb < nb_min + 64; ++nb) {
        const int band = (int)((d->H + nb - 1) / nb);
        const long long wgs = d->N * ((d->H + band - 1) / band);
        const long long cost = ((wgs + cus - 1) / cus) * ((band + 1) / 2 + 3);
        if (best < 0 || cost <= best) { best = cost; best_nb = nb; }  // ties: the split that fills more CUs
      }
      ditto::ConvRowsArgs& r = plan->cvargs;
      r.N = (int)d->N; r.C0 = (int)d->C0; r.H = (int)d->H; r.W = (int)d->W; r.C1 = (int)d->C1; r.C2 = (int)d->C2;
      r.band = (int)((d->H + best_nb - 1) / best_nb);
      r.bands = (int)((d->H + r.band - 1) / r.band);
      r.relu_mid = d->inter_op == DITTO_INTER_RELU;
      r.relu_out = d->relu_out != 0;
      plan->rows31 = true;
      plan->c1_tiles = 2;
      plan->w1p_bytes = ditto::kCvrW1Bytes;
      plan->w2p_bytes = 0;
      ditto_tile_param& t = plan->tile;
      t.block_threads = 64 * ditto::kCvrWaves;
      t.block_m = r.band * r.W;
      t.block_l = ditto::kCvrC;
      t.block_n = (int)d->C2;
      t.head_pad = ditto::kCvrC;
      t.lds_bytes = ditto::conv_rows_lds_bytes(r.W, r.band);
      t.grid_x = r.N * r.bands;
      t.grid_y = r.band;
      t.grid_z = r.W;
      t.variant = 3700 + r.band;  // row pipeline; output rows per workgroup
      return DITTO_OK;
    }
  }
  // The persistent variant (conv_chain_persist.h: W1 resident in LDS, W2 in registers, one workgroup per
  // CU walking over the tiles) is switched off: it waits for its prefetched halo tile with a hand-counted
  // `s_waitcnt vmcnt` over loads the compiler does not track, and it is slower than the kernel below
  // (33.5 against 30.5 us on 32 x 64 x 56 x 56 -> 64 -> 256).  Asking for it is refused, not ignored.
  if (steer.persist)
    return fail(DITTO_EUNSUPPORTED,
                "tile_variant %d: the persistent conv chain kernel is switched off (untracked prefetch loads; "
                "slower than the default kernel)", steer.tv);
  a.TW = (int)(Q < slots ? Q : slots);
  a.TH = slots / a.TW;
  if (a.TH > P) a.TH = (int)P;
  // Shrink the tile until the halo tile and the weight chunk fit in LDS; prefer 32-channel
  // chunks and a footprint that lets two workgroups share a CU (one stages while the other
  // computes), then 32-channel chunks alone, then 16-channel chunks.
  const int RS = a.R * a.S;
  const int th0 = a.TH, tw0 = a.TW;
  int lds = 0, ch = 32;
  for (int attempt = 0;; ++attempt) {
    ch = attempt < 2 ? 32 : 16;
    const int limit = attempt == 0 ? 78 * 1024 : 150 * 1024;
    a.TH = th0;
    a.TW = tw0;
    bool ok = false;
    for (;;) {
      a.rows_in = (a.TH - 1) * a.stride + a.R;
      a.cols_in = (a.TW - 1) * a.stride + a.S;
      lds = ditto::conv_chain_lds_bytes(a.rows_in, a.cols_in, RS, 32 * c1t, ch);
      if (lds <= limit) { ok = true; break; }
      // the first attempt only gives up rows down to half the slots
      if (a.TH > (attempt == 0 ? (th0 + 1) / 2 : 1)) a.TH = a.TH - 1;
      else if (attempt > 0 && a.TW > 16) a.TW = (a.TW + 1) / 2;
      else break;
    }
    if (ok) break;
    if (attempt == 2) return fail(DITTO_EUNSUPPORTED, "conv chain tile does not fit in LDS");
  }
  plan->ch = ch;
  plan->w1p_bytes = (size_t)ditto::conv_w1_chunk_bytes(RS, 32 * c1t, ch) * (size_t)((d->C0 + ch - 1) / ch);
  a.tiles_h = (int)((P + a.TH - 1) / a.TH);
  a.tiles_w = (int)((Q + a.TW - 1) / a.TW);
  a.relu_mid = d->inter_op == DITTO_INTER_RELU;
  a.relu_out = d->relu_out != 0;
  a.out_f32 = d->out_dtype == DITTO_F32;
  plan->c1_tiles = c1t;
  ditto_tile_param& t = plan->tile;
  t.block_threads = 256;
  t.block_m = a.TH * a.TW;   // output pixels per workgroup
  t.block_l = 32 * c1t;      // intermediate channels held in registers
  t.block_n = (int)d->C2;
  t.head_pad = ch;
  t.lds_bytes = lds;
  t.grid_x = a.N * a.tiles_h * a.tiles_w;
  t.grid_y = a.TH;
  t.grid_z = a.TW;
  t.variant = 3000 + c1t * 10 + pxw + (ch == 16 ? 100 : 0);
  return DITTO_OK;
}

}  // namespace

extern "C" {

int ditto_chain_abi_version(void) { return DITTO_CHAIN_ABI_VERSION; }

const char* ditto_last_error(void) { return g_err; }

int ditto_bmm_chain_select_tile(const ditto_bmm_chain_desc* desc, ditto_tile_param* out) {
  BmmPlan plan;
  int rc = plan_bmm(desc, &plan, true);  // the current device's compute-unit count (256 where there is none)
  if (rc != DITTO_OK) return rc;
  if (!out) return fail(DITTO_EINVAL, "null output");
  *out = plan.tile;
  return DITTO_OK;
}

size_t ditto_bmm_chain_workspace_bytes(const ditto_bmm_chain_desc* desc) {
  (void)desc;
  return 0;
}

int ditto_bmm_chain_run(const ditto_bmm_chain_desc* d, const void* a, const void* b, const void* c,
                        const void* aux, void* f, void* workspace, size_t workspace_bytes,
                        void* stream) {
  (void)workspace;
  (void)workspace_bytes;
  (void)aux;
  BmmPlan plan;
  int rc = plan_bmm(d, &plan, true);
  if (rc != DITTO_OK) return rc;
  if (!a || !b || !c || !f) return fail(DITTO_EINVAL, "null data pointer");
  if (!aligned(a, 16) || !aligned(b, 16) || !aligned(c, 16) || !aligned(f, 16))
    return fail(DITTO_EINVAL, "data pointers must be 16-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);

  if (plan.family == 0) {
    ditto::BmmChainArgs args;
    args.a = a;
    args.b = b;
    args.c = c;
    args.f = f;
    args.a_bs = d->a_batch_stride;
    args.b_bs = d->b_batch_stride;
    args.c_bs = d->c_batch_stride;
    args.f_bs = d->f_batch_stride;
    {
      const bool two = d->batch_inner > 0 && d->batch_inner != d->batch;
      args.batch_inner = two ? (int)d->batch_inner : (int)d->batch;
      args.a_bs2 = two ? d->a_batch_stride_outer : 0;
      args.b_bs2 = two ? d->b_batch_stride_outer : 0;
      args.c_bs2 = two ? d->c_batch_stride_outer : 0;
      args.f_bs2 = two ? d->f_batch_stride_outer : 0;
    }
    args.a_rs = (int)d->a_row_stride;
    args.b_rs = (int)d->b_row_stride;
    args.c_rs = (int)d->c_row_stride;
    args.f_rs = (int)d->f_row_stride;
    args.M = (int)d->M;
    args.N = (int)d->N;
    args.K = (int)d->K;
    args.L = (int)d->L;
    args.batch = (int)d->batch;
    args.mblocks = plan.nb;
    args.mblocks3 = plan.nb3;
    args.scale_log2 = d->softmax_scale * 1.4426950408889634f;
    args.relu = d->inter_op == DITTO_INTER_RELU;
    args.relu_out = d->relu_out;
    args.out_f32 = d->out_dtype == DITTO_F32;
    const bool kl = d->b_layout == DITTO_B_KL;
    const bool sm = d->inter_op == DITTO_INTER_SOFTMAX;
    hipError_t e;
    if (d->in_dtype == DITTO_F16)
      e = sm ? ditto::launch_f16_softmax(plan.d_pad, plan.qt, kl, args, st)
             : ditto::launch_f16_cast(plan.d_pad, plan.qt, kl, args, st);
    else
      e = sm ? ditto::launch_bf16_softmax(plan.d_pad, plan.qt, kl, args, st)
             : ditto::launch_bf16_cast(plan.d_pad, plan.qt, kl, args, st);
    if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
    return DITTO_OK;
  }
  if (plan.family == 1) {
    ditto::F32ChainArgs args;
    args.a = a;
    args.b = b;
    args.c = c;
    args.f = f;
    args.f64 = d->in_dtype == DITTO_F64;
    args.a_bs = d->a_batch_stride;
    args.b_bs = d->b_batch_stride;
    args.c_bs = d->c_batch_stride;
    args.f_bs = d->f_batch_stride;
    args.a_rs = (int)d->a_row_stride;
    args.b_rs = (int)d->b_row_stride;
    args.c_rs = (int)d->c_row_stride;
    args.f_rs = (int)d->f_row_stride;
    args.M = (int)d->M;
    args.N = (int)d->N;
    args.K = (int)d->K;
    args.L = (int)d->L;
    args.batch = (int)d->batch;
    args.mblocks = (int)((d->M + 31) / 32);
    args.b_lk = d->b_layout == DITTO_B_LK;
    args.relu = d->inter_op == DITTO_INTER_RELU;
    args.relu_out = d->relu_out;
    args.softmax = d->inter_op == DITTO_INTER_SOFTMAX;
    args.softmax_scale = d->softmax_scale;
    hipError_t e = ditto::launch_gemm_chain_f32(args, st);
    if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
    return DITTO_OK;
  }
  if (plan.family == 2) {
    if (aux && !aligned(aux, 4)) return fail(DITTO_EINVAL, "aux (scale vector) must be 4-byte aligned");
    ditto::I8ChainArgs args;
    args.a = static_cast<const int8_t*>(a);
    args.b = static_cast<const int8_t*>(b);
    args.d = static_cast<const int8_t*>(c);
    args.scale = static_cast<const float*>(aux);
    args.scale_uniform = d->requant_scale;
    args.wrap = d->inter_op != DITTO_INTER_REQUANT;
    args.relu = d->inter_op == DITTO_INTER_RELU;
    args.out_i8 = d->out_dtype == DITTO_I8;
    args.e = static_cast<int32_t*>(f);
    args.a_bs = d->a_batch_stride;
    args.b_bs = d->b_batch_stride;
    args.d_bs = d->c_batch_stride;
    args.e_bs = d->f_batch_stride;
    args.a_rs = (int)d->a_row_stride;
    args.b_rs = (int)d->b_row_stride;
    args.d_rs = (int)d->c_row_stride;
    args.e_rs = (int)d->f_row_stride;
    args.M = (int)d->M;
    args.N = (int)d->N;
    args.K = (int)d->K;
    args.L = (int)d->L;
    args.batch = (int)d->batch;
    args.mblocks = (int)((d->M + plan.tile.block_m - 1) / plan.tile.block_m);
    args.Lp = plan.tile.block_l;
    hipError_t e = ditto::launch_gemm_chain_i8(args, plan.d_pad, plan.qt, st);
    if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
    return DITTO_OK;
  }
  return fail(DITTO_EUNSUPPORTED, "no kernel family %d", plan.family);
}

int ditto_conv_chain_select_tile(const ditto_conv_chain_desc* desc, ditto_tile_param* out) {
  ConvPlan plan;
  int rc = plan_conv(desc, &plan, true);  // the current device's compute-unit count (256 where there is none)
  if (rc != DITTO_OK) return rc;
  if (!out) return fail(DITTO_EINVAL, "null output");
  *out = plan.tile;
  return DITTO_OK;
}

size_t ditto_conv_chain_workspace_bytes(const ditto_conv_chain_desc* desc) {
  ConvPlan plan;
  if (plan_conv(desc, &plan, true) != DITTO_OK) return 0;
  size_t need = plan.w1p_bytes + plan.w2p_bytes;
  if (plan.resident || plan.rows31 || plan.rows13) {
    // a call with pointers these kernels cannot take falls back to the general one (tile_variant 0 only): the
    // larger of the two figures, whatever the device's compute-unit count makes of the choice
    ConvPlan general;
    if (desc->tile_variant == 0 && plan_conv(desc, &general, true, 8, false) == DITTO_OK &&
        general.w1p_bytes + general.w2p_bytes > need)
      need = general.w1p_bytes + general.w2p_bytes;
  }
  return need;
}

}  // extern "C"

namespace {
// what a conv chain call does: repack the weights into the workspace, run the fused kernel, or both
enum ConvPhase { kConvPrepare = 1, kConvCompute = 2, kConvBoth = 3 };

int conv_chain_call(int phase, const ditto_conv_chain_desc* d, const void* x, const void* w1, const void* w2,
                    void* y, void* workspace, size_t workspace_bytes, void* stream) {
  ConvPlan plan;
  // (depthwise chains: 16-byte halo vectors only for a 16-byte aligned x; the tile query assumes one)
  // (the row-streaming depthwise kernel moves 16-byte vectors of x and y)
  int rc = plan_conv(d, &plan, true, x && aligned(x, 16) ? 8 : 4, true, !y || aligned(y, 16));
  if (rc != DITTO_OK) return rc;
  if (((phase & kConvCompute) && (!x || !y)) || !w1 || !w2) return fail(DITTO_EINVAL, "null data pointer");
  if (plan.resident) {
    // 16-byte direct loads of X and W1 fragments, stores of 4 pixels
    const bool ok = aligned(w1, 16) && (!(phase & kConvCompute) || (aligned(x, 16) && aligned(y, 16)));
    if (!ok && phase == kConvBoth) {
      rc = plan_conv(d, &plan, true, 4, false);  // the general kernel takes any element-aligned pointer
      if (rc != DITTO_OK) return rc;
    } else if (!ok) {
      return fail(DITTO_EINVAL, "misaligned data pointer: this shape runs with x, w1 and y 16-byte aligned "
                                "(its prepared weights are in the resident kernel's layout)");
    }
  }
  if (plan.rows13) {
    // 16-byte direct loads of X, W1 fragments and output stores; W2 as MFMA fragments in the workspace
    const bool ok = aligned(w1, 16) && workspace && workspace_bytes >= plan.w2p_bytes && aligned(workspace, 16) &&
                    (!(phase & kConvCompute) || (aligned(x, 16) && aligned(y, 16)));
    if (!ok && phase == kConvBoth) {
      rc = plan_conv(d, &plan, true, 4, false);  // the general kernel: any element-aligned pointer, workspace optional
      if (rc != DITTO_OK) return rc;
    } else if (!ok) {
      if (!workspace || workspace_bytes < plan.w2p_bytes)
        return fail(DITTO_EWORKSPACE, "prepared weights live in the workspace: need %zu bytes", plan.w2p_bytes);
      return fail(DITTO_EINVAL, "misaligned data pointer: this shape runs with x, w1, y and the workspace 16-byte "
                                "aligned (its prepared weights are in the row pipeline's layout)");
    }
  }
  if (plan.rows13) {
    ditto::ConvRowsArgs r = plan.cvargs;
    r.x = x;
    r.w1x = w1;
    r.w1f = workspace;
    r.w2 = nullptr;
    r.y = y;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const bool f16 = d->in_dtype == DITTO_F16;
    hipError_t e = hipSuccess;
    if (phase & kConvPrepare)  // W2 [C2][C1][3][3] into fragments
      e = f16 ? ditto::pack_conv_w2_resident_f16(w2, workspace, r.Cm, r.C2, st)
              : ditto::pack_conv_w2_resident_bf16(w2, workspace, r.Cm, r.C2, st);
    if (e == hipSuccess && (phase & kConvCompute))
      e = f16 ? ditto::launch_conv_rows_f16(r, st) : ditto::launch_conv_rows_bf16(r, st);
    if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
    return DITTO_OK;
  }
  if (plan.rows31) {
    // 16-byte direct loads of X, W2 fragments and output stores; W1 as MFMA fragments in the workspace
    const bool ok = aligned(w2, 16) && workspace && workspace_bytes >= plan.w1p_bytes && aligned(workspace, 16) &&
                    (!(phase & kConvCompute) || (aligned(x, 16) && aligned(y, 16)));
    if (!ok && phase == kConvBoth) {
      rc = plan_conv(d, &plan, true, 4, false);  // the general kernel: any element-aligned pointer, workspace optional
      if (rc != DITTO_OK) return rc;
    } else if (!ok) {
      if (!workspace || workspace_bytes < plan.w1p_bytes)
        return fail(DITTO_EWORKSPACE, "prepared weights live in the workspace: need %zu bytes", plan.w1p_bytes);
      return fail(DITTO_EINVAL, "misaligned data pointer: this shape runs with x, w2, y and the workspace 16-byte "
                                "aligned (its prepared weights are in the row pipeline's layout)");
    }
  }
  if (plan.rows31) {
    ditto::ConvRowsArgs r = plan.cvargs;
    r.x = x;
    r.w1f = workspace;
    r.w2 = w2;
    r.y = y;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const bool f16 = d->in_dtype == DITTO_F16;
    hipError_t e = hipSuccess;
    if (phase & kConvPrepare)  // W1 [C1][C0][3][3] into fragments: the same layout as the resident kernel's W2
      e = f16 ? ditto::pack_conv_w2_resident_f16(w1, workspace, r.C0, r.C1, st)
              : ditto::pack_conv_w2_resident_bf16(w1, workspace, r.C0, r.C1, st);
    if (e == hipSuccess && (phase & kConvCompute))
      e = f16 ? ditto::launch_conv_rows_f16(r, st) : ditto::launch_conv_rows_bf16(r, st);
    if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
    return DITTO_OK;
  }
  if (plan.resident) {
    if (!workspace) return fail(DITTO_EWORKSPACE, "this conv chain needs the workspace (%zu bytes)", plan.w2p_bytes);
    if (workspace_bytes < plan.w2p_bytes)
      return fail(DITTO_EWORKSPACE, "workspace of %zu bytes, need %zu", workspace_bytes, plan.w2p_bytes);
    if (!aligned(workspace, 16)) return fail(DITTO_EINVAL, "workspace must be 16-byte aligned");
    ditto::ConvResidentArgs r = plan.rargs;
    r.x = x;
    r.w1 = w1;
    r.w2f = workspace;
    r.y = y;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const bool f16 = d->in_dtype == DITTO_F16;
    hipError_t e = hipSuccess;
    if (phase & kConvPrepare)
      e = f16 ? ditto::pack_conv_w2_resident_f16(w2, workspace, r.C1, r.C2, st)
              : ditto::pack_conv_w2_resident_bf16(w2, workspace, r.C1, r.C2, st);
    if (e == hipSuccess && (phase & kConvCompute))
      e = f16 ? ditto::launch_conv_resident_f16(r, plan.res_grid, st) : ditto::launch_conv_resident_bf16(r, plan.res_grid, st);
    if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
    return DITTO_OK;
  }
  if (!aligned(x, 2) || !aligned(w1, 2) || !aligned(w2, 8) || !aligned(y, 4))
    return fail(DITTO_EINVAL, "misaligned data pointer");
  if (phase != kConvBoth && !plan.dw && !workspace)
    return fail(DITTO_EWORKSPACE, "prepared weights live in the workspace: none given");
  if (plan.dw) {
    if (!(phase & kConvCompute)) return DITTO_OK;  // nothing to prepare: the kernel stages the filters itself
    if (plan.dw_mode == 4) {
      ditto::DwRowsArgs r = plan.rowargs;
      r.x = x;
      r.w1 = w1;
      r.w2 = w2;
      r.y = y;
      hipStream_t st = reinterpret_cast<hipStream_t>(stream);
      hipError_t e = d->in_dtype == DITTO_F16 ? ditto::launch_dw_rows_f16(r, st) : ditto::launch_dw_rows_bf16(r, st);
      if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
      return DITTO_OK;
    }
    if (plan.dw_mode == 5) {
      ditto::Dw16RowsArgs r = plan.row16args;
      r.x = x;
      r.w1 = w1;
      r.w2 = w2;
      r.y = y;
      hipStream_t st = reinterpret_cast<hipStream_t>(stream);
      hipError_t e = d->in_dtype == DITTO_F16 ? ditto::launch_dw16_rows_f16(r, st) : ditto::launch_dw16_rows_bf16(r, st);
      if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
      return DITTO_OK;
    }
    if (!aligned(w2, 16)) return fail(DITTO_EINVAL, "misaligned data pointer");
    ditto::DwConvArgs a = plan.dwargs;
    // less aligned pointers: narrower halo loads (the LDS layout stays valid) while the chunk still
    // fits the registers that keep it in flight; plain 2-byte output stores
    while (a.vec > 1 && !aligned(x, 2 * (size_t)a.vec)) a.vec >>= 1;
    if (plan.dw_mode >= 2) {
      const int nvr = a.cols_al / a.vec;
      const int cphases = (256 * ditto::dw_mfma_groups(plan.c2_tiles) / nvr) / a.rows_in;
      if (cphases < 1 || (a.chx + cphases - 1) / cphases > (a.vec == 8 ? ditto::kDwXpf / 2 : ditto::kDwXpf))
        return fail(DITTO_EINVAL, "misaligned data pointer: x must be aligned to %d bytes for this shape",
                    2 * plan.dwargs.vec);
      if (!aligned(w1, 16)) return fail(DITTO_EINVAL, "misaligned data pointer");
    }
    if (a.wide && !aligned(y, 16)) {
      if (plan.dw_mode == 3) return fail(DITTO_EINVAL, "misaligned data pointer: y must be 16-byte aligned for this shape");
      a.wide = 0;
    }
    a.x = x;
    a.w1 = w1;
    a.w2 = w2;
    a.y = y;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    hipError_t e = d->in_dtype == DITTO_F16 ? ditto::launch_dw_conv_f16(plan.c2_tiles, plan.dw_mode, a, st)
                                            : ditto::launch_dw_conv_bf16(plan.c2_tiles, plan.dw_mode, a, st);
    if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
    return DITTO_OK;
  }
  const size_t need = plan.w1p_bytes + plan.w2p_bytes;
  if (plan.w1p_bytes >= (1ull << 31) || plan.w2p_bytes >= (1ull << 31))  // the repack kernels index with 32 bits
    return fail(DITTO_EUNSUPPORTED, "conv chain weights too large to repack");
  if (plan.px2 > 0 && !workspace)
    return fail(DITTO_EWORKSPACE, "a second convolution larger than 1x1 needs the workspace (%zu bytes)", need);
  if (workspace && workspace_bytes < need)
    return fail(DITTO_EWORKSPACE, "workspace of %zu bytes, need %zu", workspace_bytes, need);
  if (workspace && !aligned(workspace, 16)) return fail(DITTO_EINVAL, "workspace must be 16-byte aligned");
  ditto::ConvChainArgs a = plan.args;
  a.x = x;
  a.w1 = w1;
  a.w2 = w2;
  a.w1p = workspace;
  a.y = y;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool f16 = d->in_dtype == DITTO_F16;
  hipError_t e = hipSuccess;
  const bool prepare = (phase & kConvPrepare) != 0, compute = (phase & kConvCompute) != 0;
  if (workspace && plan.px2 == 0 && prepare)  // W1 into the chunked layout the chain kernel copies straight into LDS
    e = f16 ? ditto::pack_conv_w1_f16(plan.c1_tiles, plan.ch, a, workspace, st)
            : ditto::pack_conv_w1_bf16(plan.c1_tiles, plan.ch, a, workspace, st);
  if (plan.px2 > 0) {
    void* w2p = static_cast<char*>(workspace) + plan.w1p_bytes;
    a.w2p = w2p;
    if (a.wide2 && !aligned(y, 16)) a.wide2 = 0;  // plain 2-byte stores (the LDS size follows the flag)
    // both weight tensors into their chunked layouts, one launch
    if (prepare)
      e = f16 ? ditto::pack_conv_w2_f16(plan.c1_tiles, a, workspace, w2p, st)
              : ditto::pack_conv_w2_bf16(plan.c1_tiles, a, workspace, w2p, st);
    if (e == hipSuccess && compute)
      e = f16 ? ditto::launch_conv2_f16(plan.c1_tiles, plan.px2, a, st) : ditto::launch_conv2_bf16(plan.c1_tiles, plan.px2, a, st);
  } else if (e == hipSuccess && compute) {
    e = f16 ? ditto::launch_conv_f16(plan.c1_tiles, plan.ch, a, st) : ditto::launch_conv_bf16(plan.c1_tiles, plan.ch, a, st);
  }
  if (e != hipSuccess) return fail(DITTO_EHIP, "kernel launch failed: %s", hipGetErrorString(e));
  return DITTO_OK;
}

}  // namespace

extern "C" {

int ditto_conv_chain_run(const ditto_conv_chain_desc* d, const void* x, const void* w1, const void* w2,
                         void* y, void* workspace, size_t workspace_bytes, void* stream) {
  return conv_chain_call(kConvBoth, d, x, w1, w2, y, workspace, workspace_bytes, stream);
}

int ditto_conv_chain_prepare(const ditto_conv_chain_desc* d, const void* w1, const void* w2, void* workspace,
                             size_t workspace_bytes, void* stream) {
  return conv_chain_call(kConvPrepare, d, nullptr, w1, w2, nullptr, workspace, workspace_bytes, stream);
}

int ditto_conv_chain_run_prepared(const ditto_conv_chain_desc* d, const void* x, const void* w1, const void* w2,
                                  void* y, void* workspace, size_t workspace_bytes, void* stream) {
  return conv_chain_call(kConvCompute, d, x, w1, w2, y, workspace, workspace_bytes, stream);
}

}  // extern "C"

// ---- the entry point that allocates nothing -------------------------------------------------
// Its workspace (the repacked weights of a conv chain) is a file-scope device array instead of
// caller memory.  Every device the library runs on holds its own copy of the array at its own
// address until the process ends; host code reaches it only through the address taken with
// hipGetSymbolAddress on that device (the array's name is a host-side stand-in, not a device
// address).
static __device__ __align__(256) unsigned char scratch[DITTO_STATIC_WORKSPACE_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices];  // per device, filled at the first call on that device

// Device address of `scratch` on the current device.
int static_workspace(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(DITTO_EHIP, "hipGetDevice failed: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(DITTO_EUNSUPPORTED, "device ordinal %d beyond %d", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
      return fail(DITTO_EHIP, "hipGetSymbolAddress(static workspace) failed: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return DITTO_OK;
}
}  // namespace

extern "C" int ditto_conv_chain_run_static(const ditto_conv_chain_desc* d, const void* x, const void* w1,
                                           const void* w2, void* y, void* stream) {
  ConvPlan plan;
  int rc = plan_conv(d, &plan, true);
  if (rc != DITTO_OK) return rc;
  const size_t need = plan.w1p_bytes + plan.w2p_bytes;
  if (need > (size_t)DITTO_STATIC_WORKSPACE_BYTES)
    return fail(DITTO_EWORKSPACE, "the repacked weights take %zu bytes, the static workspace holds %zu", need,
                (size_t)DITTO_STATIC_WORKSPACE_BYTES);
  void* ws = nullptr;
  if (need > 0) {  // (depthwise chains stage their filters themselves and take no workspace)
    rc = static_workspace(&ws);
    if (rc != DITTO_OK) return rc;
  }
  // every byte of the workspace that the fused kernel reads is written by the repacking kernel of the
  // same call, ahead of it on `stream`: nothing has to be cleared between calls
  return conv_chain_call(kConvBoth, d, x, w1, w2, y, ws, ws ? (size_t)DITTO_STATIC_WORKSPACE_BYTES : 0, stream);
}
