// placeholder, replaced below
#include "mix_common.h"
namespace rfqmix {
bool keep_mfma_ok(int, int, int) { return false; }
void launch_attn_keep_mfma(const float*, const void*, const void*, int64_t, const int32_t*, int,
                           const int32_t*, const int32_t*, const int32_t*, const int32_t*,
                           const int32_t*, int, const float*, const void*, int64_t, void*, int64_t,
                           float, int, int, bool, int, int, int, int, int, hipStream_t) {}
}  // namespace rfqmix
