// Instantiates the fp16/bf16 chain kernel for one (element type, inter-op) pair.
// Compiled once per pair with -DDITTO_INST_T=<f16|bf16> -DDITTO_INST_INTER=<0|2>
// -DDITTO_INST_NAME=<symbol> so the variants build in parallel.
#include "bmm_chain_fp.h"

namespace ditto {

hipError_t DITTO_INST_NAME(int d_pad, int qt, bool b_kl, bool fold, const BmmChainArgs& args, hipStream_t stream) {
  typedef DITTO_INST_T T;
  constexpr int I = DITTO_INST_INTER;
#define DITTO_CASE(DP, Q)                                                          \
  if (d_pad == DP && qt == Q) {                                                    \
    if (I == kInterSoftmax && fold)                                                \
      return b_kl ? launch_bmm_chain<T, DP, Q, I, true, I == kInterSoftmax>(args, stream)   \
                  : launch_bmm_chain<T, DP, Q, I, false, I == kInterSoftmax>(args, stream); \
    return b_kl ? launch_bmm_chain<T, DP, Q, I, true, false>(args, stream)         \
                : launch_bmm_chain<T, DP, Q, I, false, false>(args, stream);       \
  }
  DITTO_CASE(64, 1)
  DITTO_CASE(64, 2)
  DITTO_CASE(128, 1)
  DITTO_CASE(128, 2)
#undef DITTO_CASE
  return hipErrorInvalidValue;
}

}  // namespace ditto
