// placeholder until the split-KV decode kernel lands
#include "common.h"
#include "device_common.h"
namespace dk {
bool decode_supported(const FwdParams &, int) { return false; }
size_t decode_workspace_bytes(const FwdParams &) { return 0; }
int launch_decode(const FwdParams &, int, void *, size_t, hipStream_t) { return fail(DK_ERR_UNSUPPORTED, "not built"); }
}  // namespace dk
