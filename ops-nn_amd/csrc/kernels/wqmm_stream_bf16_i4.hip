// Streamlined weight-only decode kernels for bf16 activations and int4 weights (one translation unit per dtype
// pair keeps the build parallel).
#include "wqmm_stream.hip.h"

namespace opsnn {
OPSNN_WQ_STREAM_DEFINE(DT_BF16, 4)
}  // namespace opsnn
