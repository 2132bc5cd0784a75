// placeholder until the MFMA forward kernel lands
#include "common.h"
#include "device_common.h"
namespace dk {
bool mfma_fwd_supported(const FwdParams &, int) { return false; }
int launch_mfma_fwd(const FwdParams &, int, hipStream_t) { return fail(DK_ERR_UNSUPPORTED, "not built"); }
}  // namespace dk
