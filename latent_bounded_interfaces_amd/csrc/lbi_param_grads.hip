// Parameter gradients of a Transformer block that are not matrix products: the RMSNorm weight and the
// depthwise causal convolution (weight and bias).  Both are sums over all rows (batch x position) with one
// result per channel, memory bound: each kernel reads its two operands once, keeps per-channel partial sums
// in registers, writes one partial vector per workgroup to the caller's workspace, and a second kernel adds
// the partials in workgroup order, so results do not depend on scheduling.
#include <hip/hip_runtime.h>

#include "lbi_common.h"

namespace lbi {
namespace param_grads {

template <typename T> __device__ __forceinline__ float round_to(float x);
template <> __device__ __forceinline__ float round_to<float>(float x) { return x; }
template <> __device__ __forceinline__ float round_to<_Float16>(float x) { return (float)(_Float16)x; }
template <> __device__ __forceinline__ float round_to<bf16_raw>(float x) {
    return __uint_as_float(((unsigned)f32_to_bf16_bits(x)) << 16);
}

constexpr int THREADS = 256;
constexpr int MAX_SLABS = 256;

// out[m] = sum over s of partials[s][m].  A workgroup takes FOLD_COLS columns; the slabs are cut into FOLD_PARTS
// contiguous ranges, one per thread of a column, each summed in ascending order, and the range sums are added in
// range order: a fixed association, whatever the launch.
constexpr int FOLD_COLS = 64, FOLD_PARTS = THREADS / FOLD_COLS;

__global__ __launch_bounds__(THREADS) void fold_partials_kernel(const float* __restrict__ partials,
                                                                float* __restrict__ out, int slabs, int width) {
    __shared__ float part_sum[FOLD_PARTS][FOLD_COLS];
    const int col = threadIdx.x % FOLD_COLS, part = threadIdx.x / FOLD_COLS;
    const int m = blockIdx.x * FOLD_COLS + col;
    const int per_part = (slabs + FOLD_PARTS - 1) / FOLD_PARTS;
    const int s_begin = part * per_part;
    const int s_end = s_begin + per_part < slabs ? s_begin + per_part : slabs;
    float acc = 0.0f;
    if (m < width) {
        int s = s_begin;
        for (; s + 8 <= s_end; s += 8) {  // eight loads in flight, added in order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partials[(size_t)(s + u) * width + m];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc += v[u];
        }
        for (; s < s_end; ++s) acc += partials[(size_t)s * width + m];
    }
    part_sum[part][col] = acc;
    __syncthreads();
    if (part == 0 && m < width) {
        float total = part_sum[0][col];
#pragma unroll
        for (int q = 1; q < FOLD_PARTS; ++q) total += part_sum[q][col];
        out[m] = total;
    }
}

inline dim3 fold_grid(int width) { return dim3((width + FOLD_COLS - 1) / FOLD_COLS); }

// ---------------------------------------------------------------------------------------
// RMSNorm weight gradient.  Forward: y = round(x_r * rsqrt(mean(x_r^2) + eps)) * weight with x_r = x rounded
// to the weight type W, so  g_weight[c] = sum over rows of g_out[row, c] * round(x_r[row, c] * r[row]).
// A wave takes one row at a time (lanes along the channels, 4 per load), a workgroup a contiguous slab of rows.
// ---------------------------------------------------------------------------------------
constexpr int NORM_MAX_VECS = 8;  // 4-channel pieces per lane: D <= 2048

template <typename W, typename X>
__global__ __launch_bounds__(THREADS) void rmsnorm_weight_grad_kernel(const W* __restrict__ g_out,
                                                                      const X* __restrict__ x,
                                                                      float* __restrict__ partials, long long rows,
                                                                      int D, float eps, int rows_per_slab) {
    extern __shared__ __align__(16) float lds[];  // [THREADS / 64][D]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int vecs = (D / 4 + 63) / 64;  // pieces per lane (some lanes hold fewer)
    float acc[NORM_MAX_VECS][4];
#pragma unroll
    for (int i = 0; i < NORM_MAX_VECS; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[i][e] = 0.0f;

    const long long row_begin = (long long)blockIdx.x * rows_per_slab;
    const long long row_end = row_begin + rows_per_slab < rows ? row_begin + rows_per_slab : rows;
    for (long long row = row_begin + wave; row < row_end; row += THREADS / 64) {
        f32x4 xr[NORM_MAX_VECS];
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < NORM_MAX_VECS; ++i) {
            const int c = 4 * lane + 256 * i;
            if (i < vecs && c < D) {
                const f32x4 v = load4(x + row * D + c);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    xr[i][e] = round_to<W>(v[e]);
                    ss = fmaf(xr[i][e], xr[i][e], ss);
                }
            }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) ss += __shfl_xor(ss, off, 64);
        const float r = rsqrtf(ss / (float)D + eps);
#pragma unroll
        for (int i = 0; i < NORM_MAX_VECS; ++i) {
            const int c = 4 * lane + 256 * i;
            if (i < vecs && c < D) {
                const f32x4 g = load4(g_out + row * D + c);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][e] = fmaf(g[e], round_to<W>(xr[i][e] * r), acc[i][e]);
            }
        }
    }
    // the four waves' sums, added in wave order
#pragma unroll
    for (int i = 0; i < NORM_MAX_VECS; ++i) {
        const int c = 4 * lane + 256 * i;
        if (i < vecs && c < D) *reinterpret_cast<f32x4*>(lds + wave * D + c) = f32x4{acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
    }
    __syncthreads();
    for (int c = threadIdx.x; c < D; c += THREADS)
        partials[(size_t)blockIdx.x * D + c] = ((lds[c] + lds[D + c]) + lds[2 * D + c]) + lds[3 * D + c];
}

inline int norm_slabs(long long rows) { return (int)(rows < MAX_SLABS ? rows : MAX_SLABS); }

template <typename W, typename X>
int launch_norm(const void* g_out, const void* x, float* out, float* partials, long long rows, int D, float eps,
                hipStream_t stream) {
    const int slabs = norm_slabs(rows);
    const int rows_per_slab = (int)((rows + slabs - 1) / slabs);
    const int used = (int)((rows + rows_per_slab - 1) / rows_per_slab);
    hipLaunchKernelGGL((rmsnorm_weight_grad_kernel<W, X>), dim3(used), dim3(THREADS), (size_t)(THREADS / 64) * D * 4,
                       stream, static_cast<const W*>(g_out), static_cast<const X*>(x), partials, rows, D, eps,
                       rows_per_slab);
    hipLaunchKernelGGL(fold_partials_kernel, fold_grid(D), dim3(THREADS), 0, stream, partials, out, used, D);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

// ---------------------------------------------------------------------------------------
// Depthwise causal convolution, weight and bias gradient.  Forward: y[b,t,c] = bias[c] + sum_j w[c,j] *
// x[b, t - (k-1-j), c] (zero before the sequence), so
//   g_w[c, j] = sum over b, t >= k-1-j of g[b,t,c] x[b, t-(k-1-j), c],   g_bias[c] = sum over b, t of g[b,t,c].
// A thread owns VEC consecutive channels and walks a slab of TS positions of one batch element, keeping the
// last k-1 inputs in registers.  Partial layout per workgroup row: [C][k] weights, then [C] bias.
// ---------------------------------------------------------------------------------------
constexpr int CONV_TS = 64;

template <typename T, int VEC, int KMAX>
__global__ __launch_bounds__(THREADS) void conv_weight_grad_kernel(const T* __restrict__ g_out,
                                                                   const T* __restrict__ x,
                                                                   float* __restrict__ partials, int T_len, int C,
                                                                   int ksize, int slabs_per_seq) {
    const int c0 = (blockIdx.x * THREADS + threadIdx.x) * VEC;
    if (c0 >= C) return;
    const int b = blockIdx.y / slabs_per_seq, slab = blockIdx.y % slabs_per_seq;
    const int t0 = slab * CONV_TS;
    const int t1 = t0 + CONV_TS < T_len ? t0 + CONV_TS : T_len;
    const size_t seq = (size_t)b * T_len;
    auto load = [&](const T* base, int t, float (&dst)[VEC]) {
        const T* p = base + (seq + t) * C + c0;
        if (VEC == 4) {
            const f32x4 v = load4(p);
#pragma unroll
            for (int e = 0; e < VEC; ++e) dst[e] = v[e];
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) dst[e] = to_f32(p[e]);
        }
    };
    float hist[KMAX][VEC];  // hist[s] = x at position t - s (s = 0 .. ksize-1); zero before the sequence
    float acc[KMAX][VEC], acc_bias[VEC];
#pragma unroll
    for (int s = 0; s < KMAX; ++s)
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            hist[s][e] = 0.0f;
            acc[s][e] = 0.0f;
        }
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc_bias[e] = 0.0f;
    // inputs just before the slab
#pragma unroll
    for (int s = 1; s < KMAX; ++s)
        if (s < ksize && t0 - s >= 0) load(x, t0 - s, hist[s - 1]);  // becomes hist[s] after the first shift
    for (int t = t0; t < t1; ++t) {
#pragma unroll
        for (int s = KMAX - 1; s >= 1; --s)
#pragma unroll
            for (int e = 0; e < VEC; ++e) hist[s][e] = hist[s - 1][e];
        load(x, t, hist[0]);
        float g[VEC];
        load(g_out, t, g);
#pragma unroll
        for (int s = 0; s < KMAX; ++s)
            if (s < ksize) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[s][e] = fmaf(g[e], hist[s][e], acc[s][e]);
            }
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc_bias[e] += g[e];
    }
    // tap j multiplies the input ksize-1-j positions back
    float* row = partials + (size_t)blockIdx.y * ((size_t)C * ksize + C);
#pragma unroll
    for (int s = 0; s < KMAX; ++s)
        if (s < ksize) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) row[(size_t)(c0 + e) * ksize + (ksize - 1 - s)] = acc[s][e];
        }
#pragma unroll
    for (int e = 0; e < VEC; ++e) row[(size_t)C * ksize + c0 + e] = acc_bias[e];
}

inline int conv_slabs_per_seq(int T_len) { return (T_len + CONV_TS - 1) / CONV_TS; }

template <typename T>
int launch_conv(const void* g_out, const void* x, float* out, float* partials, int B, int T_len, int C, int ksize,
                hipStream_t stream) {
    const int sps = conv_slabs_per_seq(T_len);
    const int slabs = B * sps;
    const int width = C * ksize + C;
    const T* gp = static_cast<const T*>(g_out);
    const T* xp = static_cast<const T*>(x);
    const bool vec4 = C % 4 == 0;
    const int per_block = THREADS * (vec4 ? 4 : 1);
    const dim3 grid((C + per_block - 1) / per_block, slabs);
    if (vec4 && ksize <= 4)
        hipLaunchKernelGGL((conv_weight_grad_kernel<T, 4, 4>), grid, dim3(THREADS), 0, stream, gp, xp, partials, T_len, C, ksize, sps);
    else if (vec4)
        hipLaunchKernelGGL((conv_weight_grad_kernel<T, 4, 8>), grid, dim3(THREADS), 0, stream, gp, xp, partials, T_len, C, ksize, sps);
    else
        hipLaunchKernelGGL((conv_weight_grad_kernel<T, 1, 8>), grid, dim3(THREADS), 0, stream, gp, xp, partials, T_len, C, ksize, sps);
    hipLaunchKernelGGL(fold_partials_kernel, fold_grid(width), dim3(THREADS), 0, stream, partials, out, slabs, width);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

}  // namespace param_grads
}  // namespace lbi

using namespace lbi;

extern "C" size_t lbi_rmsnorm_weight_grad_workspace_bytes(int64_t rows, int64_t D) {
    if (rows <= 0 || D <= 0) return 0;
    return (size_t)param_grads::norm_slabs(rows) * (size_t)D * sizeof(float);
}

extern "C" int lbi_rmsnorm_weight_grad(const void* g_out, const void* x, float* weight_grad, void* workspace,
                                       size_t workspace_bytes, int64_t rows, int64_t D, float eps, int dtype,
                                       int x_dtype, void* stream) {
    clear_error();
    if (rows < 0 || D <= 0) return fail(LBI_ERR_INVALID, "lbi_rmsnorm_weight_grad: bad size rows=%lld D=%lld", (long long)rows, (long long)D);
    if (dtype_size(dtype) == 0 || dtype_size(x_dtype) == 0)
        return fail(LBI_ERR_INVALID, "lbi_rmsnorm_weight_grad: bad dtype %d / %d", dtype, x_dtype);
    if (x_dtype != dtype && x_dtype != LBI_F32)
        return fail(LBI_ERR_UNSUPPORTED, "lbi_rmsnorm_weight_grad: x must be in the weight dtype or fp32");
    if (D % 4 != 0 || D > 256 * param_grads::NORM_MAX_VECS)
        return fail(LBI_ERR_UNSUPPORTED, "lbi_rmsnorm_weight_grad: D=%lld must be a multiple of 4, at most %d", (long long)D,
                    256 * param_grads::NORM_MAX_VECS);
    if (rows > (1ll << 40)) return fail(LBI_ERR_UNSUPPORTED, "lbi_rmsnorm_weight_grad: too many rows");
    if (!weight_grad) return fail(LBI_ERR_INVALID, "lbi_rmsnorm_weight_grad: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (rows == 0) {  // an empty sum: zeros, written by the fold kernel (no partials are read)
        hipLaunchKernelGGL(param_grads::fold_partials_kernel, param_grads::fold_grid((int)D),
                           dim3(param_grads::THREADS), 0, s, static_cast<const float*>(nullptr), weight_grad, 0, (int)D);
        LBI_HIP_CHECK(hipGetLastError());
        return LBI_OK;
    }
    if (!g_out || !x) return fail(LBI_ERR_INVALID, "lbi_rmsnorm_weight_grad: null pointer");
    const size_t need = lbi_rmsnorm_weight_grad_workspace_bytes(rows, D);
    if (!workspace || workspace_bytes < need)
        return fail(LBI_ERR_WORKSPACE, "lbi_rmsnorm_weight_grad: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    const size_t align_g = dtype_size(dtype) * 4, align_x = dtype_size(x_dtype) * 4;
    if (reinterpret_cast<uintptr_t>(g_out) % align_g || reinterpret_cast<uintptr_t>(x) % align_x ||
        reinterpret_cast<uintptr_t>(workspace) % 16)
        return fail(LBI_ERR_INVALID, "lbi_rmsnorm_weight_grad: misaligned pointer");
    float* ws = static_cast<float*>(workspace);
    const bool wide_x = x_dtype == LBI_F32;
    switch (dtype) {
        case LBI_F32: return param_grads::launch_norm<float, float>(g_out, x, weight_grad, ws, rows, (int)D, eps, s);
        case LBI_F16:
            return wide_x ? param_grads::launch_norm<_Float16, float>(g_out, x, weight_grad, ws, rows, (int)D, eps, s)
                          : param_grads::launch_norm<_Float16, _Float16>(g_out, x, weight_grad, ws, rows, (int)D, eps, s);
        default:
            return wide_x ? param_grads::launch_norm<bf16_raw, float>(g_out, x, weight_grad, ws, rows, (int)D, eps, s)
                          : param_grads::launch_norm<bf16_raw, bf16_raw>(g_out, x, weight_grad, ws, rows, (int)D, eps, s);
    }
}

extern "C" size_t lbi_causal_conv1d_weight_grad_workspace_bytes(int64_t B, int64_t T, int64_t C, int64_t ksize) {
    if (B <= 0 || T <= 0 || C <= 0 || ksize <= 0) return 0;
    return (size_t)B * (size_t)param_grads::conv_slabs_per_seq((int)T) * ((size_t)C * ksize + C) * sizeof(float);
}

extern "C" int lbi_causal_conv1d_weight_grad(const void* g_out, const void* x, float* grads, void* workspace,
                                             size_t workspace_bytes, int64_t B, int64_t T, int64_t C, int64_t ksize,
                                             int dtype, void* stream) {
    clear_error();
    if (B < 0 || T < 0 || C <= 0 || ksize <= 0)
        return fail(LBI_ERR_INVALID, "lbi_causal_conv1d_weight_grad: bad size B=%lld T=%lld C=%lld k=%lld", (long long)B,
                    (long long)T, (long long)C, (long long)ksize);
    if (dtype_size(dtype) == 0) return fail(LBI_ERR_INVALID, "lbi_causal_conv1d_weight_grad: bad dtype %d", dtype);
    if (ksize > 8) return fail(LBI_ERR_UNSUPPORTED, "lbi_causal_conv1d_weight_grad: kernel sizes above 8 are not supported");
    if (B > (1 << 20) || T > (1 << 24) || C > (1 << 20) || (double)B * T > 6.0e4 * param_grads::CONV_TS)
        return fail(LBI_ERR_UNSUPPORTED, "lbi_causal_conv1d_weight_grad: size out of range");
    if (!grads) return fail(LBI_ERR_INVALID, "lbi_causal_conv1d_weight_grad: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (B == 0 || T == 0) {  // an empty sum: zeros, written by the fold kernel (no partials are read)
        const int width = (int)(C * ksize + C);
        hipLaunchKernelGGL(param_grads::fold_partials_kernel, param_grads::fold_grid(width),
                           dim3(param_grads::THREADS), 0, s, static_cast<const float*>(nullptr), grads, 0, width);
        LBI_HIP_CHECK(hipGetLastError());
        return LBI_OK;
    }
    if (!g_out || !x) return fail(LBI_ERR_INVALID, "lbi_causal_conv1d_weight_grad: null pointer");
    const size_t need = lbi_causal_conv1d_weight_grad_workspace_bytes(B, T, C, ksize);
    if (!workspace || workspace_bytes < need)
        return fail(LBI_ERR_WORKSPACE, "lbi_causal_conv1d_weight_grad: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    const size_t align = C % 4 == 0 ? dtype_size(dtype) * 4 : dtype_size(dtype);
    if (reinterpret_cast<uintptr_t>(g_out) % align || reinterpret_cast<uintptr_t>(x) % align ||
        reinterpret_cast<uintptr_t>(workspace) % 4)
        return fail(LBI_ERR_INVALID, "lbi_causal_conv1d_weight_grad: misaligned pointer");
    float* ws = static_cast<float*>(workspace);
    switch (dtype) {
        case LBI_F32: return param_grads::launch_conv<float>(g_out, x, grads, ws, (int)B, (int)T, (int)C, (int)ksize, s);
        case LBI_F16: return param_grads::launch_conv<_Float16>(g_out, x, grads, ws, (int)B, (int)T, (int)C, (int)ksize, s);
        default: return param_grads::launch_conv<bf16_raw>(g_out, x, grads, ws, (int)B, (int)T, (int)C, (int)ksize, s);
    }
}
