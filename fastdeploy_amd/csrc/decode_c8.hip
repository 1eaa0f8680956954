// placeholder until the MFMA kernel lands
#include "fdattn_common.h"
namespace fdattn {
size_t c8_workspace_bytes(int, int) { return 0; }
bool c8_supported(int, int, int, int, int) { return false; }
int decode_c8_launch(const void*, const void*, const void*, const float*, const float*, const int32_t*,
                     const int32_t*, const int32_t*, const int32_t*, const int32_t*, int, void*, void*, size_t,
                     int, int, int, int, int, int, int, int, float, hipStream_t) {
  return fail(FDATTN_ERR_SHAPE, "decode_c8: not built");
}
}  // namespace fdattn
