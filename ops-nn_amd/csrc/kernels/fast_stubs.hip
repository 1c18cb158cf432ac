// Placeholder until each MFMA family lands in its own file.
#include "common.hip.h"
#include "launch.h"
namespace opsnn {
int launch_blockscale_mfma(const OpsnnQmmArgs&, hipStream_t) { return OPSNN_NOT_TAKEN; }
int launch_mx_mfma(const OpsnnQmmArgs&, hipStream_t) { return OPSNN_NOT_TAKEN; }
int launch_wqmm_mfma(const OpsnnWqmmArgs&, hipStream_t) { return OPSNN_NOT_TAKEN; }
}
