// Instantiates the row pipeline of the conv3x3 -> conv1x1 chain for one element type.
// Compiled with -DDITTO_INST_T=<f16|bf16> and -DDITTO_CONVROWS_NAME=<symbol>.
#include "conv_rows.h"

namespace ditto {

// 3x3 (pad 1, stride 1) -> 1x1 with at most 64 -> 64 -> 256 channels, image rows of at most 64 pixels
hipError_t DITTO_CONVROWS_NAME(const ConvRowsArgs& args, hipStream_t stream) {
  return launch_conv_rows<DITTO_INST_T>(args, stream);
}

}  // namespace ditto
