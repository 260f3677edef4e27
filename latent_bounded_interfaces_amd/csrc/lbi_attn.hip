// Attention input-pullback for P cotangent basis directions (gfx950): C ABI entry points
// and the choice between the MFMA kernels and the generic kernels.
#include "lbi_attn_generic.h"
#include "lbi_attn_mfma.h"
#include "lbi_attn_dkdv128.h"
#include "lbi_attn_dkdv_pair.h"
#include "lbi_attn_dq128.h"
#include "lbi_attn_small.h"

#include <cstdlib>
#include <mutex>

namespace lbi {
namespace {

// Scratch memory of lbi_attn_pullback_static: one copy per GPU the library runs on, held until the process ends.
// In host code this name only stands for the symbol; the device address comes from hipGetSymbolAddress, once per
// device, and only that pointer is ever handed to a kernel.
static __device__ __align__(256) unsigned char scratch[LBI_ATTN_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
std::atomic<void*> g_scratch_ptr[kMaxDevices];  // zero-initialised

// Device address of `scratch` on the current device.  Looked up on the first call per device (under a lock, with
// hipGetSymbolAddress); every later call reads the kept pointer and makes no runtime call but hipGetDevice.
int static_scratch(void** out) {
    int device = -1;
    LBI_HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices)
        return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_pullback_static: device index %d out of range", device);
    void* ptr = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!ptr) {
        std::lock_guard<std::mutex> guard(g_scratch_mutex);
        ptr = g_scratch_ptr[device].load(std::memory_order_relaxed);
        if (!ptr) {
            LBI_HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
            if (!ptr) return fail(LBI_ERR_HIP, "lbi_attn_pullback_static: scratch symbol has no device address");
            g_scratch_ptr[device].store(ptr, std::memory_order_release);
        }
    }
    *out = ptr;
    return LBI_OK;
}

int check_attn_dims(int64_t B, int64_t H, int64_t T, int64_t Dh, int64_t P, int dtype) {
    if (B < 0 || H < 0 || T < 0 || Dh < 0 || P < 0)
        return fail(LBI_ERR_INVALID, "lbi_attn_pullback: negative size (B=%lld H=%lld T=%lld Dh=%lld P=%lld)",
                    (long long)B, (long long)H, (long long)T, (long long)Dh, (long long)P);
    if (dtype != LBI_F32 && dtype != LBI_F16 && dtype != LBI_BF16)
        return fail(LBI_ERR_INVALID, "lbi_attn_pullback: dtype must be float, half or bfloat16 (got %d)", dtype);
    if (B > (1 << 20) || H > (1 << 16) || T > (1 << 24) || Dh > (1 << 16) || P > (1 << 16) ||
        (double)B * H * T * Dh * (P > 1 ? P : 1) > 1.0e15 || (double)B * H * (P > 1 ? P : 1) > 2.0e9)
        return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_pullback: size out of range");
    return LBI_OK;
}

// Short sequences: one launch that does everything per (b, h, direction), no workspace.  LBI_ATTN_SMALL=0 keeps
// the four-kernel path.
bool use_small_path(int T_len, int dh, int dtype) {
    static const bool enabled = !(std::getenv("LBI_ATTN_SMALL") && std::atoi(std::getenv("LBI_ATTN_SMALL")) == 0);
    return enabled && attn_small::supports(T_len, dh, dtype);
}

}  // namespace
}  // namespace lbi

extern "C" size_t lbi_attn_pullback_workspace_bytes(int64_t B, int64_t H, int64_t T, int64_t Dh, int64_t P,
                                                    int dtype) {
    using namespace lbi;
    if (check_attn_dims(B, H, T, Dh, P, dtype) != LBI_OK) return 0;
    if (B == 0 || H == 0 || T == 0 || Dh == 0 || P == 0) return 0;
    if (use_small_path((int)T, (int)Dh, dtype)) return 0;
    const size_t floats = attn_mfma::supports((int)T, (int)Dh, dtype) ? attn_mfma::workspace_floats(B, H, T, Dh, P)
                                                                     : attn_generic::workspace_floats(B, H, T, P);
    return (floats * sizeof(float) + 255) & ~(size_t)255;
}

extern "C" int lbi_attn_pullback(const void* q, const void* k, const void* v, const void* d_out, void* dq, void* dk,
                                 void* dv, void* workspace, size_t workspace_bytes, int64_t B, int64_t H, int64_t T,
                                 int64_t Dh, int64_t P, float softmax_scale, int causal, int dtype, void* stream_v) {
    using namespace lbi;
    clear_error();
    if (int rc = check_attn_dims(B, H, T, Dh, P, dtype)) return rc;
    if (B == 0 || H == 0 || T == 0 || Dh == 0 || P == 0) return LBI_OK;
    if (!q || !k || !v || !d_out || !dq || !dk || !dv) return fail(LBI_ERR_INVALID, "lbi_attn_pullback: null tensor pointer");
    const size_t need = lbi_attn_pullback_workspace_bytes(B, H, T, Dh, P, dtype);
    if (need > 0 && (!workspace || workspace_bytes < need))
        return fail(LBI_ERR_WORKSPACE, "lbi_attn_pullback: workspace of %zu bytes needed, %zu given", need,
                    workspace_bytes);
    if (need > 0 && reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return fail(LBI_ERR_WORKSPACE, "lbi_attn_pullback: workspace must be 16-byte aligned");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    float* ws = static_cast<float*>(workspace);
    const int b = (int)B, h = (int)H, t = (int)T, dh = (int)Dh, p = (int)P;
    if (use_small_path(t, dh, dtype)) {
        const size_t align = dtype_size(dtype) * 8;
        if (reinterpret_cast<uintptr_t>(q) % align || reinterpret_cast<uintptr_t>(k) % align ||
            reinterpret_cast<uintptr_t>(v) % align || reinterpret_cast<uintptr_t>(d_out) % align ||
            reinterpret_cast<uintptr_t>(dq) % 8 || reinterpret_cast<uintptr_t>(dk) % 8 ||
            reinterpret_cast<uintptr_t>(dv) % 8)
            return fail(LBI_ERR_INVALID, "lbi_attn_pullback: tensors must be 16-byte aligned");
        return dtype == LBI_F16
                   ? attn_small::launch<_Float16>(q, k, v, d_out, dq, dk, dv, b, h, t, dh, p, softmax_scale, causal, stream)
                   : attn_small::launch<bf16_raw>(q, k, v, d_out, dq, dk, dv, b, h, t, dh, p, softmax_scale, causal, stream);
    }
    if (attn_mfma::supports(t, dh, dtype)) {
        const size_t align = dtype_size(dtype) * 8;  // 16-byte vector loads on every row
        if (reinterpret_cast<uintptr_t>(q) % align || reinterpret_cast<uintptr_t>(k) % align ||
            reinterpret_cast<uintptr_t>(v) % align || reinterpret_cast<uintptr_t>(d_out) % align)
            return fail(LBI_ERR_INVALID, "lbi_attn_pullback: tensors must be 16-byte aligned");
        return dtype == LBI_F16
                   ? attn_mfma::launch<_Float16>(q, k, v, d_out, dq, dk, dv, ws, b, h, t, dh, p, softmax_scale, causal, stream)
                   : attn_mfma::launch<bf16_raw>(q, k, v, d_out, dq, dk, dv, ws, b, h, t, dh, p, softmax_scale, causal, stream);
    }
    switch (dtype) {
        case LBI_F32: return attn_generic::launch<float>(q, k, v, d_out, dq, dk, dv, ws, b, h, t, dh, p, softmax_scale, causal, stream);
        case LBI_F16: return attn_generic::launch<_Float16>(q, k, v, d_out, dq, dk, dv, ws, b, h, t, dh, p, softmax_scale, causal, stream);
        default: return attn_generic::launch<bf16_raw>(q, k, v, d_out, dq, dk, dv, ws, b, h, t, dh, p, softmax_scale, causal, stream);
    }
}

extern "C" int lbi_attn_pullback_static(const void* q, const void* k, const void* v, const void* d_out, void* dq,
                                        void* dk, void* dv, int64_t B, int64_t H, int64_t T, int64_t Dh, int64_t P,
                                        float softmax_scale, int causal, int dtype, void* stream_v) {
    using namespace lbi;
    clear_error();
    if (int rc = check_attn_dims(B, H, T, Dh, P, dtype)) return rc;
    if (B == 0 || H == 0 || T == 0 || Dh == 0 || P == 0) return LBI_OK;
    if (!q || !k || !v || !d_out || !dq || !dk || !dv)
        return fail(LBI_ERR_INVALID, "lbi_attn_pullback_static: null tensor pointer");
    const size_t need = lbi_attn_pullback_workspace_bytes(B, H, T, Dh, P, dtype);
    if (need > (size_t)LBI_ATTN_STATIC_SCRATCH_BYTES)
        return fail(LBI_ERR_WORKSPACE,
                    "lbi_attn_pullback_static: this call needs %zu bytes of scratch memory, the static buffer holds %zu; "
                    "use lbi_attn_pullback with a caller-provided workspace",
                    need, (size_t)LBI_ATTN_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if (need > 0)
        if (int rc = static_scratch(&ws)) return rc;
    // Every kernel of the pullback writes its part of the workspace before any kernel reads it, so what the last
    // call left behind needs no clearing.
    return lbi_attn_pullback(q, k, v, d_out, dq, dk, dv, ws, need, B, H, T, Dh, P, softmax_scale, causal, dtype,
                             stream_v);
}
