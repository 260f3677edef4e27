// Attention input-pullback for P cotangent basis directions (gfx950).
#include "lbi_common.h"

extern "C" size_t lbi_attn_pullback_workspace_bytes(int64_t, int64_t, int64_t, int64_t, int64_t, int) { return 0; }

extern "C" int lbi_attn_pullback(const void*, const void*, const void*, const void*, void*, void*, void*, void*,
                                 size_t, int64_t, int64_t, int64_t, int64_t, int64_t, float, int, int, void*) {
    return lbi::fail(LBI_ERR_UNSUPPORTED, "lbi_attn_pullback: not built yet");
}
