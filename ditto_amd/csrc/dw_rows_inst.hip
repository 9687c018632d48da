// Instantiates the row-streaming depthwise chain kernel for one element type.
// Compiled with -DDITTO_INST_T=<f16|bf16> and -DDITTO_DWROWS_NAME=<symbol>.
#include "dw_rows.h"

namespace ditto {

// depthwise 3x3 (multiplier 1) -> 1x1 with at most 32 -> 64 channels, image rows of at most 128 pixels
hipError_t DITTO_DWROWS_NAME(const DwRowsArgs& args, hipStream_t stream) {
  return launch_dw_rows<DITTO_INST_T>(args, stream);
}

}  // namespace ditto
