// Frobenius and spectral norms of a batch of square matrices (the Jacobian diagnostics of the
// interface scan), without a singular value decomposition.
//
// sigma_1(A) = ||A||_F * sqrt(lambda_1(G_0)),  G_0 = X^T X,  X = A / ||A||_F.
// The top eigenvalue of the symmetric positive semidefinite G_0 comes from repeated squaring with the
// trace divided out each time:  Gh_k = G_k / tr(G_k),  G_{k+1} = Gh_k^2,  so
//   log lambda_1(G_0) = log t_0 + 1/2 log t_1 + 1/4 log t_2 + ... + 2^-n log lambda_1(Gh_n),  t_k = tr(G_k).
// lambda_1(Gh_n) lies in [q, sqrt(q)] with q = ||Gh_n||_F^2 <= 1, and q -> 1 as Gh_n approaches rank one, so the
// last term is bounded by 2^-n log(d): after the 24 squarings allowed here the estimate is exact to fp32
// rounding whatever the spectrum; well-separated spectra stop after a handful of squarings.
//
// One workgroup per matrix (grid-stride over the batch).  The two d x d fp32 buffers live in LDS when they
// fit in 64 KB (d <= 88: scalar products), otherwise in a per-workgroup slice of the caller's workspace (L2
// resident), padded to a multiple of 32 so that the products run on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32): the Gram matrix is then X X^T, which has the same top eigenvalue as X^T X, both
// operands are row strips, and only the tiles on and above the diagonal are formed and mirrored.
#include "lbi_common.h"

namespace lbi {
namespace norms {

constexpr int THREADS = 256;
constexpr int MAX_SQUARINGS = 24;
constexpr int LDS_LIMIT_BYTES = 64 * 1024;

inline bool fits_lds(int ld) { return 2ll * ld * ld * 4 <= LDS_LIMIT_BYTES; }
// leading dimension of the buffers: a multiple of 4 in LDS, of 32 (matrix-core tiles) in the workspace
inline int padded(int d) {
    const int ld4 = (d + 3) & ~3;
    return fits_lds(ld4) ? ld4 : (d + 31) & ~31;
}
inline int grid_for(long long n, int ld) {
    const long long cap = ld <= 256 ? 1024 : 256;
    return (int)(n < cap ? n : cap);
}

__device__ __forceinline__ float block_sum(float x, float* red) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
    __syncthreads();  // red may still be read by the previous call's consumers; also publishes buffer writes
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = x;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < THREADS / 64; ++w) total += red[w];
    return total;
}

// H = X^T X for ld x ld row-major X (ld a multiple of 4); each thread forms 4 x 4 tiles.  For symmetric X
// this is X^2.  Rows k of X are read as two 16-byte pieces, so both operands stream along rows.
__device__ __forceinline__ void gram(const float* X, float* H, int ld) {
    const int tiles = ld >> 2;
    for (int tile = threadIdx.x; tile < tiles * tiles; tile += THREADS) {
        const int i0 = (tile / tiles) << 2, j0 = (tile % tiles) << 2;
        float acc[4][4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[r][c] = 0.0f;
#pragma unroll 4
        for (int k = 0; k < ld; ++k) {
            const f32x4 a = *reinterpret_cast<const f32x4*>(X + (long long)k * ld + i0);
            const f32x4 b = *reinterpret_cast<const f32x4*>(X + (long long)k * ld + j0);
#pragma unroll
            for (int r = 0; r < 4; ++r)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[r][c] = fmaf(a[r], b[c], acc[r][c]);
        }
#pragma unroll
        for (int r = 0; r < 4; ++r)
            *reinterpret_cast<f32x4*>(H + (long long)(i0 + r) * ld + j0) = f32x4{acc[r][0], acc[r][1], acc[r][2], acc[r][3]};
    }
}

// H = X X^T for ld x ld row-major X, ld a multiple of 32, on the fp32 matrix cores (for symmetric X this is X^2).
// Tile (ti, tj), ti <= tj, is sum_k X[32 ti + m][k] X[32 tj + n][k]: both operands are 16-byte pieces of rows (a lane
// of half h takes k = 8 q + 4 h + e for the e-th product of piece q, the same on both sides).  The tiles on and
// above the diagonal are dealt to the four waves in turn; each is written twice, so H is exactly symmetric.
// `scale` multiplies the result (the normalisation of X folded into the product: (cX)(cX)^T = c^2 X X^T).
__device__ __forceinline__ void gram_mfma(const float* X, float* H, int ld, float scale) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, m = lane & 31, h = lane >> 5;
    const int nt = ld >> 5;
    int turn = 0;
    for (int ti = 0; ti < nt; ++ti)
        for (int tj = ti; tj < nt; ++tj, ++turn) {
            if ((turn & 3) != wave) continue;
            const float* a_row = X + (long long)(32 * ti + m) * ld + 4 * h;
            const float* b_row = X + (long long)(32 * tj + m) * ld + 4 * h;
            f32x16 acc;
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[e] = 0.0f;
#pragma unroll 4
            for (int q = 0; q < ld / 8; ++q) {
                const f32x4 a = *reinterpret_cast<const f32x4*>(a_row + 8 * q);
                const f32x4 b = *reinterpret_cast<const f32x4*>(b_row + 8 * q);
#pragma unroll
                for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e] * scale, b[e], acc, 0, 0, 0);
            }
            // register 4 g + e of lane (m, h) is row 8 g + 4 h + e, column m of the tile
#pragma unroll
            for (int g = 0; g < 4; ++g) {
#pragma unroll
                for (int e = 0; e < 4; ++e) H[(long long)(32 * ti + 8 * g + 4 * h + e) * ld + 32 * tj + m] = acc[4 * g + e];
                if (ti != tj)
                    *reinterpret_cast<f32x4*>(H + (long long)(32 * tj + m) * ld + 32 * ti + 8 * g + 4 * h) =
                        f32x4{acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
            }
        }
}

template <typename T>
__global__ __launch_bounds__(THREADS) void matrix_norms_kernel(const T* __restrict__ mats, float* __restrict__ spectral,
                                                               float* __restrict__ frobenius, float* scratch, long long n,
                                                               int d, int ld, int use_lds) {
    extern __shared__ __align__(16) float lds_buffers[];
    __shared__ float red[THREADS / 64];
    const long long plane = (long long)ld * ld;
    float* buf0 = use_lds ? lds_buffers : scratch + (long long)blockIdx.x * 2 * plane;
    float* buf1 = buf0 + plane;

    for (long long m = blockIdx.x; m < n; m += gridDim.x) {
        const T* a = mats + m * (long long)d * d;
        float ss = 0.0f;
        for (int idx = threadIdx.x; idx < (int)plane; idx += THREADS) {
            const int r = idx / ld, c = idx - r * ld;
            const float v = (r < d && c < d) ? to_f32(a[(long long)r * d + c]) : 0.0f;
            buf0[idx] = v;
            ss = fmaf(v, v, ss);
        }
        ss = block_sum(ss, red);
        const float fro = sqrtf(ss);
        if (!(ss > 0.0f) || !(fro < __builtin_inff())) {  // zero matrix, overflow or NaN: both norms are `fro`
            if (threadIdx.x == 0) {
                frobenius[m] = fro;
                spectral[m] = fro;
            }
            __syncthreads();
            continue;
        }
        const float inv = 1.0f / fro;
        for (int idx = threadIdx.x; idx < (int)plane; idx += THREADS) buf0[idx] *= inv;
        __syncthreads();

        float* x = buf0;
        float* h = buf1;
        if (use_lds) gram(x, h, ld);
        else gram_mfma(x, h, ld, 1.0f);
        float log_lambda = 0.0f, weight = 1.0f;
        for (int step = 0;; ++step) {
            float tr = 0.0f;  // block_sum's first barrier publishes h
            __syncthreads();
            for (int i = threadIdx.x; i < ld; i += THREADS) tr += h[(long long)i * ld + i];
            tr = block_sum(tr, red);
            const float inv_tr = 1.0f / tr;
            float q = 0.0f;
            if (use_lds) {
                for (int idx = threadIdx.x; idx < (int)plane; idx += THREADS) {
                    const float v = h[idx] * inv_tr;
                    h[idx] = v;
                    q = fmaf(v, v, q);
                }
            } else {  // h stays as it is: the next product takes the factor, this pass only reads
                for (int idx = 4 * threadIdx.x; idx < (int)plane; idx += 4 * THREADS) {
                    const f32x4 v = *reinterpret_cast<const f32x4*>(h + idx);
                    q = fmaf(v[0], v[0], fmaf(v[1], v[1], fmaf(v[2], v[2], fmaf(v[3], v[3], q))));
                }
                q *= inv_tr * inv_tr;
            }
            q = block_sum(q, red);
            log_lambda += weight * logf(tr);
            if (q >= 1.0f - 1e-7f || step == MAX_SQUARINGS || !(q > 0.0f)) {
                if (q > 0.0f) log_lambda += weight * 0.75f * logf(fminf(q, 1.0f));  // middle of [q, sqrt(q)] in logs
                break;
            }
            __syncthreads();  // h fully scaled before it becomes the operand
            float* t = x;
            x = h;
            h = t;
            if (use_lds) gram(x, h, ld);
            else gram_mfma(x, h, ld, inv_tr * inv_tr);
            weight *= 0.5f;
        }
        if (threadIdx.x == 0) {
            frobenius[m] = fro;
            spectral[m] = fro * expf(0.5f * log_lambda);
        }
        __syncthreads();  // buffers are reused by the next matrix
    }
}

template <typename T>
int launch(const void* mats, float* spectral, float* frobenius, void* workspace, long long n, int d, hipStream_t stream) {
    const int ld = padded(d);
    const bool use_lds = fits_lds(ld);
    const size_t lds_bytes = use_lds ? (size_t)2 * ld * ld * 4 : 0;
    hipLaunchKernelGGL((matrix_norms_kernel<T>), dim3(grid_for(n, ld)), dim3(THREADS), lds_bytes, stream, (const T*)mats,
                       spectral, frobenius, (float*)workspace, n, d, ld, use_lds ? 1 : 0);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

}  // namespace norms
}  // namespace lbi

using namespace lbi;

extern "C" size_t lbi_matrix_norms_workspace_bytes(int64_t N, int64_t d) {
    if (N <= 0 || d <= 0 || d > 2048) return 0;
    const int ld = norms::padded((int)d);
    if (norms::fits_lds(ld)) return 0;
    return (size_t)norms::grid_for(N, ld) * 2 * ld * ld * sizeof(float);
}

extern "C" int lbi_matrix_norms(const void* mats, float* spectral, float* frobenius, void* workspace,
                                size_t workspace_bytes, int64_t N, int64_t d, int dtype, void* stream) {
    clear_error();
    if (N < 0 || d <= 0 || d > 2048) return fail(LBI_ERR_INVALID, "lbi_matrix_norms: bad size N=%lld d=%lld (d in 1..2048)", (long long)N, (long long)d);
    if (dtype_size(dtype) == 0) return fail(LBI_ERR_INVALID, "lbi_matrix_norms: bad dtype %d", dtype);
    if (N == 0) return LBI_OK;
    if (!mats || !spectral || !frobenius) return fail(LBI_ERR_INVALID, "lbi_matrix_norms: null pointer");
    const size_t need = lbi_matrix_norms_workspace_bytes(N, d);
    if (need > 0 && (!workspace || workspace_bytes < need))
        return fail(LBI_ERR_WORKSPACE, "lbi_matrix_norms: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    if (need > 0 && reinterpret_cast<uintptr_t>(workspace) % 16 != 0)
        return fail(LBI_ERR_INVALID, "lbi_matrix_norms: workspace must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case LBI_F32: return norms::launch<float>(mats, spectral, frobenius, workspace, N, (int)d, s);
        case LBI_F16: return norms::launch<_Float16>(mats, spectral, frobenius, workspace, N, (int)d, s);
        default: return norms::launch<bf16_raw>(mats, spectral, frobenius, workspace, N, (int)d, s);
    }
}
