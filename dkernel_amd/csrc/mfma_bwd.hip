// placeholder until the MFMA backward kernels land
#include "common.h"
#include "device_common.h"
namespace dk {
bool mfma_bwd_supported(const BwdParams &, int) { return false; }
int launch_mfma_bwd(const BwdParams &, int, hipStream_t) { return fail(DK_ERR_UNSUPPORTED, "not built"); }
}  // namespace dk
