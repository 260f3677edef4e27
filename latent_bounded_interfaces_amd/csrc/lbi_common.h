// Shared host/device helpers for the gfx950 kernels of liblbi_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/lbi_hip.h"

namespace lbi {

// Records a printf-style message for lbi_last_error() on the calling thread and
// returns `status`, so failing paths read `return fail(LBI_ERR_INVALID, "...")`.
int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
void clear_error();

inline size_t dtype_size(int dtype) {
    return dtype == LBI_F32 ? 4 : (dtype == LBI_F16 || dtype == LBI_BF16) ? 2 : 0;
}

#define LBI_HIP_CHECK(expr)                                                              \
    do {                                                                                 \
        hipError_t lbi_e_ = (expr);                                                      \
        if (lbi_e_ != hipSuccess)                                                        \
            return ::lbi::fail(LBI_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(lbi_e_)); \
    } while (0)

// Raises the dynamic-LDS limit of kernel KERN to `bytes` where the default 64 KiB does not do.  The runtime call is
// made once per kernel and device (a later, larger request raises it again); launches after that only read a flag,
// so nothing but the launch itself happens on a hot path or inside a stream capture.  A failure is reported, not
// left for the launch to trip over.
template <auto KERN>
int ensure_dynamic_lds(size_t bytes) {
    constexpr int kTracked = 32;
    static std::atomic<size_t> granted[kTracked];  // zero-initialised
    if (bytes <= 64 * 1024) return LBI_OK;
    int dev = 0;
    LBI_HIP_CHECK(hipGetDevice(&dev));
    const bool tracked = dev >= 0 && dev < kTracked;
    if (tracked && granted[dev].load(std::memory_order_relaxed) >= bytes) return LBI_OK;
    LBI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(KERN), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (int)bytes));
    if (tracked) granted[dev].store(bytes, std::memory_order_relaxed);
    return LBI_OK;
}

// Compute units of the current device, asked of the runtime once per device and kept (256 on a whole MI355X, 32 per
// partition when the part is split into its XCDs); 256 if the runtime will not say.  Launch plans that weigh "how
// many workgroups fill the chip" use this figure.  The workgroup -> XCD dealing of the kernels (ids equal mod 8
// share an L2) assumes the eight XCDs of an unpartitioned gfx950 part and is merely a permutation otherwise.
inline int device_compute_units() {
    constexpr int kTracked = 32;
    static std::atomic<int> known[kTracked];  // zero-initialised
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kTracked) return 256;
    int cus = known[dev].load(std::memory_order_relaxed);
    if (cus > 0) return cus;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
    known[dev].store(cus, std::memory_order_relaxed);
    return cus;
}

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x4 __attribute__((ext_vector_type(4)));
typedef unsigned short u16x8 __attribute__((ext_vector_type(8)));

// Storage element types. bf16 is carried as raw 16-bit words and widened by a
// shift, which is exact.
struct bf16_raw { unsigned short bits; };

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(_Float16 x) { return (float)x; }
__device__ __forceinline__ float to_f32(bf16_raw x) { return __uint_as_float(((unsigned)x.bits) << 16); }

// Round-to-nearest-even narrowing (NaN stays a quiet NaN): the hardware conversion, v_cvt_pk_bf16_f32.
__device__ __forceinline__ unsigned short f32_to_bf16_bits(float x) {
    return __builtin_bit_cast(unsigned short, (__bf16)x);
}

// Four consecutive storage elements widened to fp32 with one vector load.
// `p` must be aligned to 4 elements.
__device__ __forceinline__ f32x4 load4(const float* p) { return *reinterpret_cast<const f32x4*>(p); }
__device__ __forceinline__ f32x4 load4(const _Float16* p) {
    f16x4 h = *reinterpret_cast<const f16x4*>(p);
    return f32x4{(float)h[0], (float)h[1], (float)h[2], (float)h[3]};
}
__device__ __forceinline__ f32x4 load4(const bf16_raw* p) {
    u16x4 h = *reinterpret_cast<const u16x4*>(p);
    return f32x4{__uint_as_float(((unsigned)h[0]) << 16), __uint_as_float(((unsigned)h[1]) << 16),
                 __uint_as_float(((unsigned)h[2]) << 16), __uint_as_float(((unsigned)h[3]) << 16)};
}

}  // namespace lbi
