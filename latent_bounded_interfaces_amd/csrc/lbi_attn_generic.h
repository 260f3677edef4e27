// Attention input-pullback, generic path: any T, any head dim <= 256, any storage
// type, causal or not.  Scalar fp32 arithmetic on 16 x 16 tiles staged in LDS.
// This is the path for fp32 inputs and for shapes the MFMA kernels do not take;
// it is not tuned.
//
// Workspace layout (floats): lse2[B*H*T] (log2-domain logsumexp), delta[B*P*H*T].
#pragma once

#include "lbi_common.h"

namespace lbi {
namespace attn_generic {

constexpr int TILE = 16;
constexpr int MAX_DH = 256;
constexpr int MAX_ACC = MAX_DH / TILE;
constexpr float LOG2E = 1.4426950408889634f;

template <typename T> __device__ __forceinline__ void store_elem(T* p, float v);
template <> __device__ __forceinline__ void store_elem<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_elem<_Float16>(_Float16* p, float v) { *p = (_Float16)v; }
template <> __device__ __forceinline__ void store_elem<bf16_raw>(bf16_raw* p, float v) { p->bits = f32_to_bf16_bits(v); }

// Cooperative load of up to TILE rows x dh elements (rows >= T are zero) into LDS, pitch dh+1.
template <typename T>
__device__ __forceinline__ void load_tile(float* dst, const T* src, int row0, int T_len, int dh, int tid) {
    for (int idx = tid; idx < TILE * dh; idx += 256) {
        const int r = idx / dh;
        const int c = idx % dh;
        const int row = row0 + r;
        dst[r * (dh + 1) + c] = row < T_len ? to_f32(src[(size_t)row * dh + c]) : 0.0f;
    }
}

__device__ __forceinline__ float dot_rows(const float* a, const float* b, int dh) {
    float acc = 0.0f;
    for (int c = 0; c < dh; ++c) acc = fmaf(a[c], b[c], acc);
    return acc;
}

// Sum over the 16 lanes that share a tile row (lanes tid%16 = 0..15 are consecutive).
__device__ __forceinline__ float row_sum16(float v) {
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) v += __shfl_xor(v, off, 16);
    return v;
}
__device__ __forceinline__ float row_max16(float v) {
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 16));
    return v;
}

// lse2[b,h,i] = log2(sum_j exp(scale * q_i . k_j)) over the keys row i may see.
template <typename T>
__global__ __launch_bounds__(256) void lse_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                  float* __restrict__ lse2, int T_len, int dh, float scale,
                                                  int causal) {
    extern __shared__ float smem[];
    float* qs = smem;
    float* ks = qs + TILE * (dh + 1);
    const int tid = threadIdx.x;
    const int r = tid / TILE, c = tid % TILE;
    const int i0 = blockIdx.x * TILE;
    const size_t bh = blockIdx.y;
    const T* q_bh = q + bh * (size_t)T_len * dh;
    const T* k_bh = k + bh * (size_t)T_len * dh;
    load_tile(qs, q_bh, i0, T_len, dh, tid);
    const int i = i0 + r;
    const int j_end = causal ? min(T_len, i0 + TILE) : T_len;
    const float sc2 = scale * LOG2E;
    float m_run = -INFINITY, l_run = 0.0f;
    for (int j0 = 0; j0 < j_end; j0 += TILE) {
        __syncthreads();
        load_tile(ks, k_bh, j0, T_len, dh, tid);
        __syncthreads();
        const int j = j0 + c;
        const bool valid = j < T_len && (!causal || j <= i);
        if (valid) {
            const float s = dot_rows(qs + r * (dh + 1), ks + c * (dh + 1), dh) * sc2;
            const float m_new = fmaxf(m_run, s);
            l_run = l_run * exp2f(m_run - m_new) + exp2f(s - m_new);
            m_run = m_new;
        }
    }
    const float m_all = row_max16(m_run);
    const float l_all = row_sum16(m_run == -INFINITY ? 0.0f : l_run * exp2f(m_run - m_all));
    if (c == 0 && i < T_len) lse2[bh * T_len + i] = m_all + log2f(l_all);
}

// delta[b,p,h,i] = sum_j P_ij * (d_out_p,i . v_j)
template <typename T>
__global__ __launch_bounds__(256) void delta_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                    const T* __restrict__ v, const T* __restrict__ d_out,
                                                    const float* __restrict__ lse2, float* __restrict__ delta,
                                                    int H, int P, int T_len, int dh, float scale, int causal) {
    extern __shared__ float smem[];
    const int pitch = dh + 1;
    float* qs = smem;
    float* gs = qs + TILE * pitch;
    float* ks = gs + TILE * pitch;
    float* vs = ks + TILE * pitch;
    const int tid = threadIdx.x;
    const int r = tid / TILE, c = tid % TILE;
    const int i0 = blockIdx.x * TILE;
    const int bph = blockIdx.y;  // (b*P + p)*H + h
    const int h = bph % H, p = (bph / H) % P, b = bph / (H * P);
    const size_t bh = (size_t)b * H + h;
    const size_t row_base = bh * T_len;
    const T* q_bh = q + row_base * dh;
    const T* k_bh = k + row_base * dh;
    const T* v_bh = v + row_base * dh;
    const T* g_bph = d_out + (size_t)bph * T_len * dh;
    load_tile(qs, q_bh, i0, T_len, dh, tid);
    load_tile(gs, g_bph, i0, T_len, dh, tid);
    const int i = i0 + r;
    const float my_lse = i < T_len ? lse2[row_base + i] : 0.0f;
    const int j_end = causal ? min(T_len, i0 + TILE) : T_len;
    const float sc2 = scale * LOG2E;
    float acc = 0.0f;
    for (int j0 = 0; j0 < j_end; j0 += TILE) {
        __syncthreads();
        load_tile(ks, k_bh, j0, T_len, dh, tid);
        load_tile(vs, v_bh, j0, T_len, dh, tid);
        __syncthreads();
        const int j = j0 + c;
        if (i < T_len && j < T_len && (!causal || j <= i)) {
            const float prob = exp2f(dot_rows(qs + r * pitch, ks + c * pitch, dh) * sc2 - my_lse);
            acc = fmaf(prob, dot_rows(gs + r * pitch, vs + c * pitch, dh), acc);
        }
    }
    acc = row_sum16(acc);
    if (c == 0 && i < T_len) delta[(size_t)bph * T_len + i] = acc;
}

// dq[b,p,h,i,:] = scale * sum_j dS_ij k_j
template <typename T>
__global__ __launch_bounds__(256) void dq_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                 const T* __restrict__ v, const T* __restrict__ d_out,
                                                 const float* __restrict__ lse2, const float* __restrict__ delta,
                                                 T* __restrict__ dq, int H, int P, int T_len, int dh, float scale,
                                                 int causal) {
    extern __shared__ float smem[];
    const int pitch = dh + 1;
    float* qs = smem;
    float* gs = qs + TILE * pitch;
    float* ks = gs + TILE * pitch;
    float* vs = ks + TILE * pitch;
    float* dss = vs + TILE * pitch;  // [TILE][TILE+1]
    const int tid = threadIdx.x;
    const int r = tid / TILE, c = tid % TILE;
    const int i0 = blockIdx.x * TILE;
    const int bph = blockIdx.y;
    const int h = bph % H, b = bph / (H * P);
    const size_t bh = (size_t)b * H + h;
    const size_t row_base = bh * T_len;
    const T* k_bh = k + row_base * dh;
    const T* v_bh = v + row_base * dh;
    load_tile(qs, q + row_base * dh, i0, T_len, dh, tid);
    load_tile(gs, d_out + (size_t)bph * T_len * dh, i0, T_len, dh, tid);
    const int i = i0 + r;
    const float my_lse = i < T_len ? lse2[row_base + i] : 0.0f;
    const float my_delta = i < T_len ? delta[(size_t)bph * T_len + i] : 0.0f;
    const int j_end = causal ? min(T_len, i0 + TILE) : T_len;
    const float sc2 = scale * LOG2E;
    float acc[MAX_ACC];
#pragma unroll
    for (int a = 0; a < MAX_ACC; ++a) acc[a] = 0.0f;
    for (int j0 = 0; j0 < j_end; j0 += TILE) {
        __syncthreads();
        load_tile(ks, k_bh, j0, T_len, dh, tid);
        load_tile(vs, v_bh, j0, T_len, dh, tid);
        __syncthreads();
        const int j = j0 + c;
        float ds = 0.0f;
        if (i < T_len && j < T_len && (!causal || j <= i)) {
            const float prob = exp2f(dot_rows(qs + r * pitch, ks + c * pitch, dh) * sc2 - my_lse);
            ds = prob * (dot_rows(gs + r * pitch, vs + c * pitch, dh) - my_delta);
        }
        dss[r * (TILE + 1) + c] = ds;
        __syncthreads();
#pragma unroll
        for (int a = 0; a < MAX_ACC; ++a) {
            const int d = c + a * TILE;
            if (d < dh) {
                float s = acc[a];
#pragma unroll
                for (int jj = 0; jj < TILE; ++jj) s = fmaf(dss[r * (TILE + 1) + jj], ks[jj * pitch + d], s);
                acc[a] = s;
            }
        }
    }
    if (i < T_len) {
        T* dst = dq + ((size_t)bph * T_len + i) * dh;
#pragma unroll
        for (int a = 0; a < MAX_ACC; ++a) {
            const int d = c + a * TILE;
            if (d < dh) store_elem(dst + d, acc[a] * scale);
        }
    }
}

// dk[b,p,h,j,:] = scale * sum_i dS_ij q_i ;  dv[b,p,h,j,:] = sum_i P_ij d_out_p,i
template <typename T>
__global__ __launch_bounds__(256) void dkdv_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                   const T* __restrict__ v, const T* __restrict__ d_out,
                                                   const float* __restrict__ lse2, const float* __restrict__ delta,
                                                   T* __restrict__ dk, T* __restrict__ dv, int H, int P, int T_len,
                                                   int dh, float scale, int causal) {
    extern __shared__ float smem[];
    const int pitch = dh + 1;
    float* qs = smem;
    float* gs = qs + TILE * pitch;
    float* ks = gs + TILE * pitch;
    float* vs = ks + TILE * pitch;
    float* dss = vs + TILE * pitch;       // [query][key]
    float* pss = dss + TILE * (TILE + 1);  // [query][key]
    const int tid = threadIdx.x;
    const int r = tid / TILE, c = tid % TILE;
    const int j0 = blockIdx.x * TILE;
    const int bph = blockIdx.y;
    const int h = bph % H, b = bph / (H * P);
    const size_t bh = (size_t)b * H + h;
    const size_t row_base = bh * T_len;
    const T* q_bh = q + row_base * dh;
    const T* g_bph = d_out + (size_t)bph * T_len * dh;
    load_tile(ks, k + row_base * dh, j0, T_len, dh, tid);
    load_tile(vs, v + row_base * dh, j0, T_len, dh, tid);
    const float sc2 = scale * LOG2E;
    float acc_k[MAX_ACC], acc_v[MAX_ACC];
#pragma unroll
    for (int a = 0; a < MAX_ACC; ++a) acc_k[a] = acc_v[a] = 0.0f;
    // In phase 1 a thread is (query r, key c); in phase 2 it is (key r, dims c + 16a).
    for (int i0 = causal ? j0 : 0; i0 < T_len; i0 += TILE) {
        __syncthreads();
        load_tile(qs, q_bh, i0, T_len, dh, tid);
        load_tile(gs, g_bph, i0, T_len, dh, tid);
        __syncthreads();
        const int i = i0 + r;
        const int j = j0 + c;
        float prob = 0.0f, ds = 0.0f;
        if (i < T_len && j < T_len && (!causal || j <= i)) {
            prob = exp2f(dot_rows(qs + r * pitch, ks + c * pitch, dh) * sc2 - lse2[row_base + i]);
            ds = prob * (dot_rows(gs + r * pitch, vs + c * pitch, dh) - delta[(size_t)bph * T_len + i]);
        }
        pss[r * (TILE + 1) + c] = prob;
        dss[r * (TILE + 1) + c] = ds;
        __syncthreads();
#pragma unroll
        for (int a = 0; a < MAX_ACC; ++a) {
            const int d = c + a * TILE;
            if (d < dh) {
                float sk = acc_k[a], sv = acc_v[a];
#pragma unroll
                for (int ii = 0; ii < TILE; ++ii) {
                    sk = fmaf(dss[ii * (TILE + 1) + r], qs[ii * pitch + d], sk);
                    sv = fmaf(pss[ii * (TILE + 1) + r], gs[ii * pitch + d], sv);
                }
                acc_k[a] = sk;
                acc_v[a] = sv;
            }
        }
    }
    const int j = j0 + r;
    if (j < T_len) {
        T* dst_k = dk + ((size_t)bph * T_len + j) * dh;
        T* dst_v = dv + ((size_t)bph * T_len + j) * dh;
#pragma unroll
        for (int a = 0; a < MAX_ACC; ++a) {
            const int d = c + a * TILE;
            if (d < dh) {
                store_elem(dst_k + d, acc_k[a] * scale);
                store_elem(dst_v + d, acc_v[a]);
            }
        }
    }
}

inline size_t workspace_floats(int64_t B, int64_t H, int64_t T, int64_t P) { return (size_t)(B * H * T + B * P * H * T); }

template <typename T>
int launch(const void* q, const void* k, const void* v, const void* d_out, void* dq, void* dk, void* dv,
           float* workspace, int B, int H, int T_len, int dh, int P, float scale, int causal, hipStream_t stream) {
    if (dh > MAX_DH) return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_pullback: head dim %d > %d", dh, MAX_DH);
    float* lse2 = workspace;
    float* delta = workspace + (size_t)B * H * T_len;
    const int tiles = (T_len + TILE - 1) / TILE;
    const size_t tile_bytes = (size_t)TILE * (dh + 1) * sizeof(float);
    const size_t sq_bytes = (size_t)TILE * (TILE + 1) * sizeof(float);
    const T* qp = static_cast<const T*>(q);
    const T* kp = static_cast<const T*>(k);
    const T* vp = static_cast<const T*>(v);
    const T* gp = static_cast<const T*>(d_out);
    if ((size_t)B * H > 65535 || (size_t)B * H * P > 65535)
        return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_pullback: B*H*P too large for the generic path");
    hipLaunchKernelGGL(lse_kernel<T>, dim3(tiles, B * H), dim3(256), 2 * tile_bytes, stream, qp, kp, lse2, T_len, dh,
                       scale, causal);
    hipLaunchKernelGGL(delta_kernel<T>, dim3(tiles, B * P * H), dim3(256), 4 * tile_bytes, stream, qp, kp, vp, gp,
                       lse2, delta, H, P, T_len, dh, scale, causal);
    hipLaunchKernelGGL(dq_kernel<T>, dim3(tiles, B * P * H), dim3(256), 4 * tile_bytes + sq_bytes, stream, qp, kp, vp,
                       gp, lse2, delta, static_cast<T*>(dq), H, P, T_len, dh, scale, causal);
    hipLaunchKernelGGL(dkdv_kernel<T>, dim3(tiles, B * P * H), dim3(256), 4 * tile_bytes + 2 * sq_bytes, stream, qp,
                       kp, vp, gp, lse2, delta, static_cast<T*>(dk), static_cast<T*>(dv), H, P, T_len, dh, scale,
                       causal);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

}  // namespace attn_generic
}  // namespace lbi
