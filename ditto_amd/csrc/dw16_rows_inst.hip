// Instantiates the row-streaming depthwise chain kernel for sixteen outputs per input channel, one element type.
// Compiled with -DDITTO_INST_T=<f16|bf16> and -DDITTO_DW16ROWS_NAME=<symbol>.
#include "dw16_rows.h"

namespace ditto {

// depthwise 3x3 (multiplier 16) -> 1x1 with at most 32 -> 512 -> 64 channels, image rows of at most 120 pixels
hipError_t DITTO_DW16ROWS_NAME(const Dw16RowsArgs& args, hipStream_t stream) {
  return launch_dw16_rows<DITTO_INST_T>(args, stream);
}

}  // namespace ditto
