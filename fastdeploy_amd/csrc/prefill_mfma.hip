// placeholder until the MFMA prefill kernel lands
#include "fdattn_common.h"
namespace fdattn {
struct PrefillArgs;
bool prefill_mfma_supported(int, int, int, int, int) { return false; }
int prefill_mfma_launch(const PrefillArgs&, int, int, hipStream_t) { return fail(FDATTN_ERR_SHAPE, "not built"); }
}  // namespace fdattn
