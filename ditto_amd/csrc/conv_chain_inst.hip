// Instantiates the conv chain kernel for one element type.
// Compiled with -DDITTO_INST_T=<f16|bf16> -DDITTO_INST_NAME=<symbol>.
#include "conv_chain.h"

namespace ditto {

hipError_t DITTO_INST_NAME(int c1_tiles, const ConvChainArgs& args, hipStream_t stream) {
  typedef DITTO_INST_T T;
  switch (c1_tiles) {
    case 1:
      return launch_conv_chain<T, 1, 2>(args, stream);
    case 2:
      return launch_conv_chain<T, 2, 2>(args, stream);
    case 4:
      return launch_conv_chain<T, 4, 2>(args, stream);
    case 8:
      return launch_conv_chain<T, 8, 1>(args, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace ditto
