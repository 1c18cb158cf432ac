// Placeholder until each MFMA family lands in its own file.
#include "common.hip.h"
#include "launch.h"
namespace opsnn {
int launch_wqmm_mfma(const OpsnnWqmmArgs&, hipStream_t) { return OPSNN_NOT_TAKEN; }
}
