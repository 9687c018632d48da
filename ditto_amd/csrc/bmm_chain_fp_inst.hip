// Instantiates the fp16/bf16 chain kernels for one (element type, inter-op) pair.
// Compiled once per pair with -DDITTO_INST_T=<f16|bf16> -DDITTO_INST_INTER=<0|2>
// -DDITTO_INST_NAME=<symbol> so the variants build in parallel.
#include "bmm_chain_fp8.h"
#include "bmm_chain_fp8m16.h"
#include "bmm_chain_fp4m16.h"

namespace ditto {

// q = 1 | 2: four-wave kernel, 32*q rows per wave; q = 8: eight-wave kernel; q = 9: eight-wave kernel,
// software pipelined; q = 6 | 7: eight-wave kernel on the 16x16x32 MFMA (7: args.mblocks3 of a
// batch entry's row blocks have 384 rows); q = 4 | 5: four-wave kernel on the 16x16x32 MFMA, 64-row workgroups (head_pad 64;
// 5: the waves split the keys of a tile as well as the rows)
hipError_t DITTO_INST_NAME(int d_pad, int q, bool b_kl, const BmmChainArgs& args, hipStream_t stream) {
  typedef DITTO_INST_T T;
  constexpr int I = DITTO_INST_INTER;
#define DITTO_CASE(DP, Q)                                                  \
  if (d_pad == DP && q == Q)                                               \
    return b_kl ? launch_bmm_chain<T, DP, Q, I, true>(args, stream)        \
                : launch_bmm_chain<T, DP, Q, I, false>(args, stream);
#define DITTO_CASE8(DP)                                                    \
  if (d_pad == DP && q == 8)                                               \
    return b_kl ? launch_bmm_chain8<T, DP, I, true>(args, stream)          \
                : launch_bmm_chain8<T, DP, I, false>(args, stream);
#define DITTO_CASE9(DP)                                                    \
  if (d_pad == DP && q == 9)                                               \
    return b_kl ? launch_bmm_chain8<T, DP, I, true, true>(args, stream)    \
                : launch_bmm_chain8<T, DP, I, false, true>(args, stream);
#define DITTO_CASE6(DP)                                                    \
  if (d_pad == DP && (q == 6 || q == 7))                                   \
    return b_kl ? launch_bmm_chain8m16<T, DP, I, true>(args, stream) : launch_bmm_chain8m16<T, DP, I, false>(args, stream);
  if (d_pad == 64 && q == 4)
    return b_kl ? launch_bmm_chain4m16<T, 64, I, 1, true>(args, stream) : launch_bmm_chain4m16<T, 64, I, 1, false>(args, stream);
  if (d_pad == 64 && q == 5)
    return b_kl ? launch_bmm_chain4m16<T, 64, I, 2, true>(args, stream) : launch_bmm_chain4m16<T, 64, I, 2, false>(args, stream);
  DITTO_CASE(64, 1)
  DITTO_CASE(64, 2)
  DITTO_CASE(128, 1)
  DITTO_CASE(128, 2)
  DITTO_CASE8(64)
  DITTO_CASE8(128)
  DITTO_CASE9(64)
  DITTO_CASE9(128)
  DITTO_CASE6(64)
  DITTO_CASE6(128)
#undef DITTO_CASE
#undef DITTO_CASE8
#undef DITTO_CASE9
#undef DITTO_CASE6
  return hipErrorInvalidValue;
}

}  // namespace ditto
