// placeholder; replaced by the tuned kernels
#include "bp_common.h"
namespace bp {
bool mfma_supports(const GemmArgs&) { return false; }
int launch_mfma(const GemmArgs&, hipStream_t) { return BP_ERR_UNSUPPORTED; }
}
