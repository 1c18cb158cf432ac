// Streamlined weight-only decode kernels for f16 activations and int8 weights (one translation unit per dtype
// pair keeps the build parallel).
#include "wqmm_stream.hip.h"

namespace opsnn {
OPSNN_WQ_STREAM_DEFINE(DT_F16, 8)
}  // namespace opsnn
