// Attention input-pullback for short sequences in one launch (fp16 / bf16 storage; any T up to 256 at head dim
// 64 and up to 128 at head dim 128).
//
// At these sizes a call is bound by launch and pipeline-fill latency, not by arithmetic, so one
// workgroup does everything for one (b, h, direction): Q, K, V and d_out_p (T x Dh each) are
// copied to LDS once, and the four waves run two passes over them.  A wave owns tile w of 32 rows and, when
// there are more than four tiles, also tile 7 - w, which evens out the causal work.
//   pass 1, per owned tile of 32 queries (lanes = queries, registers = keys, as in the dQ kernel):
//     S^T = K Q^T, softmax over the wave's registers, dP^T = V dO^T, delta = sum_j P dP,
//     dS = P (dP - delta), dQ = scale dS K; the row statistics (log-sum-exp, delta) go to LDS
//   pass 2, per owned tile of 32 keys (lanes = keys, registers = queries, as in the dK/dV kernel):
//     S = Q K^T, P = exp2(S c - lse), dP = dO V^T, dS = P (dP - delta),
//     dV = P^T dO, dK = scale dS^T Q
// A length that is no multiple of 32 fills its last tile with zero rows: as keys they are masked out (the causal
// mask already does that), as queries they carry a zero cotangent and add nothing; their outputs are not stored.
// Every output tile has one owner and every sum a fixed order: reruns are bit-identical.
#pragma once

#include "lbi_attn_mfma.h"

namespace lbi {
namespace attn_small {

using namespace attn_mfma;

// Q, K, V, d_out (MAX_TILES tiles of 32 x DH each), then lse2[32 MAX_TILES], delta[32 MAX_TILES]
template <int DH, int MAX_TILES> constexpr size_t lds_bytes() {
    return (size_t)4 * MAX_TILES * 32 * DH * 2 + (size_t)2 * 32 * MAX_TILES * sizeof(float);
}
static_assert(lds_bytes<64, 8>() <= 160 * 1024 && lds_bytes<128, 4>() <= 160 * 1024, "LDS budget");

inline int max_seq(int dh) { return dh == 64 ? 256 : (dh == 128 ? 128 : 0); }
inline bool supports(int T_len, int dh, int dtype) {
    return (dtype == LBI_F16 || dtype == LBI_BF16) && T_len >= 1 && T_len <= max_seq(dh);
}

// Four values of one output row (consecutive head-dim elements), scaled, as 8 bytes.
template <typename T>
__device__ __forceinline__ void store4(T* dst, const f32x16& c, int g, float scale) {
    *reinterpret_cast<u32x2*>(dst) = u32x2{Mma<T>::pack2(c[4 * g] * scale, c[4 * g + 1] * scale),
                                           Mma<T>::pack2(c[4 * g + 2] * scale, c[4 * g + 3] * scale)};
}

// Two workgroups per CU where LDS allows it (head dim 64 up to 128 positions).
template <typename T, int DH, int MAX_TILES, bool CAUSAL>
__global__ __launch_bounds__(256, (DH == 64 && MAX_TILES == 4) ? 2 : 1) void small_seq_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                        const T* __restrict__ v, const T* __restrict__ d_out,
                                                        T* __restrict__ dq, T* __restrict__ dk, T* __restrict__ dv,
                                                        int n_bh, int H, int P, int T_len, float scale) {
    constexpr int KS = DH / 16, ND = DH / 32, TILE_BYTES = 32 * DH * 2, OPERAND_BYTES = MAX_TILES * TILE_BYTES;
    constexpr int MAX_T = 32 * MAX_TILES, OWNED = MAX_TILES / 4;
    static_assert(MAX_TILES == 4 || MAX_TILES == 8, "a wave owns one or two tiles");
    extern __shared__ __align__(16) char smem[];
    char* q_lds = smem;
    char* k_lds = smem + OPERAND_BYTES;
    char* v_lds = smem + 2 * OPERAND_BYTES;
    char* g_lds = smem + 3 * OPERAND_BYTES;
    float* lse_lds = reinterpret_cast<float*>(smem + 4 * OPERAND_BYTES);
    float* delta_lds = lse_lds + MAX_T;

    int bh, p;
    if (!map_block(P, n_bh, bh, p)) return;
    const int nt = (T_len + 31) / 32;  // 1 .. MAX_TILES; the last tile may be partly past the end
    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int b = bh / H, hh = bh - b * H;
    const size_t base = (size_t)bh * T_len * DH;                               // q, k, v
    const size_t gbase = (((size_t)b * P + p) * H + hh) * (size_t)T_len * DH;  // d_out, dq, dk, dv
    const float sc2 = scale * LOG2E;

    {
        // rows past the end of the sequence (last tile of a ragged length) are zero
        auto fetch = [&](TileLoader<DH>& ld, const T* src, int row0) __attribute__((always_inline)) {
            constexpr int CPR = DH / 8;
#pragma unroll
            for (int u = 0; u < TileLoader<DH>::N; ++u) {
                const int id = tid + 256 * u;
                const int r = row0 + id / CPR, c = id % CPR;
                ld.regs[u] = r < T_len ? *reinterpret_cast<const u32x4*>(src + (size_t)r * DH + c * 8) : u32x4{0u, 0u, 0u, 0u};
            }
        };
        TileLoader<DH> lq[MAX_TILES], lk[MAX_TILES], lv[MAX_TILES], lg[MAX_TILES];
#pragma unroll
        for (int t = 0; t < MAX_TILES; ++t)
            if (t < nt) {
                fetch(lq[t], q + base, 32 * t);
                fetch(lk[t], k + base, 32 * t);
                fetch(lv[t], v + base, 32 * t);
                fetch(lg[t], d_out + gbase, 32 * t);
            }
#pragma unroll
        for (int t = 0; t < MAX_TILES; ++t)
            if (t < nt) {
                lq[t].commit(q_lds + t * TILE_BYTES, tid);
                lk[t].commit(k_lds + t * TILE_BYTES, tid);
                lv[t].commit(v_lds + t * TILE_BYTES, tid);
                lg[t].commit(g_lds + t * TILE_BYTES, tid);
            }
    }
    __syncthreads();

    // ---- pass 1: each owned tile of 32 queries against every key tile it may see
#pragma unroll 1
    for (int own = 0; own < OWNED; ++own) {
        const int qt = own == 0 ? wave : MAX_TILES - 1 - wave;
        if (qt >= nt) continue;  // those 32 rows do not exist
        const int jt_end = CAUSAL ? qt + 1 : nt;
        u32x4 qf[KS], gf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            qf[ks] = frag_nat<DH>(q_lds + qt * TILE_BYTES, m, h, ks);
            gf[ks] = frag_nat<DH>(g_lds + qt * TILE_BYTES, m, h, ks);
        }
        f32x16 s[MAX_TILES], dp[MAX_TILES];
        float row_max = -INFINITY;
#pragma unroll
        for (int jt = 0; jt < MAX_TILES; ++jt)
            if (jt < jt_end) {
                s[jt] = zero16();
                dp[jt] = zero16();
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) s[jt] = Mma<T>::mma(frag_nat<DH>(k_lds + jt * TILE_BYTES, m, h, ks), qf[ks], s[jt]);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) dp[jt] = Mma<T>::mma(frag_nat<DH>(v_lds + jt * TILE_BYTES, m, h, ks), gf[ks], dp[jt]);
                const bool diag = CAUSAL && jt == qt;
                const int keys_left = T_len - 32 * jt;  // < 32 only in a ragged last tile
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    float x = s[jt][r] * sc2;
                    if (diag && c_row(r, h) > m) x = -INFINITY;  // key after the query
                    if (!CAUSAL && c_row(r, h) >= keys_left) x = -INFINITY;  // key past the end
                    s[jt][r] = x;
                    row_max = fmaxf(row_max, x);
                }
            }
        row_max = fmaxf(row_max, __shfl_xor(row_max, 32, 64));
        float row_sum = 0.0f;
#pragma unroll
        for (int jt = 0; jt < MAX_TILES; ++jt)
            if (jt < jt_end) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float e = __builtin_amdgcn_exp2f(s[jt][r] - row_max);
                    s[jt][r] = e;
                    row_sum += e;
                }
            }
        row_sum += __shfl_xor(row_sum, 32, 64);
        const float inv = 1.0f / row_sum;
        float delta = 0.0f;
#pragma unroll
        for (int jt = 0; jt < MAX_TILES; ++jt)
            if (jt < jt_end) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    s[jt][r] *= inv;
                    delta = fmaf(s[jt][r], dp[jt][r], delta);
                }
            }
        delta += __shfl_xor(delta, 32, 64);
        f32x16 dq_t[ND];
#pragma unroll
        for (int nd = 0; nd < ND; ++nd) dq_t[nd] = zero16();
#pragma unroll
        for (int jt = 0; jt < MAX_TILES; ++jt)
            if (jt < jt_end) {
#pragma unroll
                for (int r = 0; r < 16; ++r) dp[jt][r] = s[jt][r] * (dp[jt][r] - delta);
#pragma unroll
                for (int kk = 0; kk < 2; ++kk) {
                    const u32x4 ds_frag = pack_frag<T>(dp[jt], kk);
#pragma unroll
                    for (int nd = 0; nd < ND; ++nd)
                        dq_t[nd] = Mma<T>::mma(frag_tr<DH>(k_lds + jt * TILE_BYTES, lane, 16 * kk, 32 * nd), ds_frag, dq_t[nd]);
                }
            }
        if (32 * qt + m < T_len) {
            T* dq_row = dq + gbase + (size_t)(32 * qt + m) * DH;
#pragma unroll
            for (int nd = 0; nd < ND; ++nd)
#pragma unroll
                for (int g = 0; g < 4; ++g) store4<T>(dq_row + 32 * nd + 8 * g + 4 * h, dq_t[nd], g, scale);
        }
        if (h == 0) {
            lse_lds[32 * qt + m] = row_max + log2f(row_sum);
            delta_lds[32 * qt + m] = delta;
        }
    }
    __syncthreads();

    // ---- pass 2: each owned tile of 32 keys against every query tile that may see them
#pragma unroll 1
    for (int own = 0; own < OWNED; ++own) {
        const int kt = own == 0 ? wave : MAX_TILES - 1 - wave;
        if (kt >= nt) continue;
        u32x4 kf[KS], vf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            kf[ks] = frag_nat<DH>(k_lds + kt * TILE_BYTES, m, h, ks);
            vf[ks] = frag_nat<DH>(v_lds + kt * TILE_BYTES, m, h, ks);
        }
        f32x16 dk_t[ND], dv_t[ND];
#pragma unroll
        for (int nd = 0; nd < ND; ++nd) {
            dk_t[nd] = zero16();
            dv_t[nd] = zero16();
        }
#pragma unroll 1
        for (int it = CAUSAL ? kt : 0; it < nt; ++it) {
            const char* q_tile = q_lds + it * TILE_BYTES;
            const char* g_tile = g_lds + it * TILE_BYTES;
            f32x16 s = zero16(), dp = zero16();
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) s = Mma<T>::mma(frag_nat<DH>(q_tile, m, h, ks), kf[ks], s);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) dp = Mma<T>::mma(frag_nat<DH>(g_tile, m, h, ks), vf[ks], dp);
            const bool diag = CAUSAL && it == kt;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                // registers 4g .. 4g+3 are queries 32 it + 8g + 4h + (0 .. 3)
                const f32x4 lse4 = *reinterpret_cast<const f32x4*>(lse_lds + 32 * it + 8 * g + 4 * h);
                const f32x4 del4 = *reinterpret_cast<const f32x4*>(delta_lds + 32 * it + 8 * g + 4 * h);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int r = 4 * g + e;
                    float pr = __builtin_amdgcn_exp2f(s[r] * sc2 - lse4[e]);
                    if (diag && m > c_row(r, h)) pr = 0.0f;  // key after the query
                    s[r] = pr;
                    dp[r] = pr * (dp[r] - del4[e]);
                }
            }
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const u32x4 p_frag = pack_frag<T>(s, kk);
                const u32x4 ds_frag = pack_frag<T>(dp, kk);
#pragma unroll
                for (int nd = 0; nd < ND; ++nd) {
                    dv_t[nd] = Mma<T>::mma(frag_tr<DH>(g_tile, lane, 16 * kk, 32 * nd), p_frag, dv_t[nd]);
                    dk_t[nd] = Mma<T>::mma(frag_tr<DH>(q_tile, lane, 16 * kk, 32 * nd), ds_frag, dk_t[nd]);
                }
            }
        }
        if (32 * kt + m < T_len) {
            T* dk_row = dk + gbase + (size_t)(32 * kt + m) * DH;
            T* dv_row = dv + gbase + (size_t)(32 * kt + m) * DH;
#pragma unroll
            for (int nd = 0; nd < ND; ++nd)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    store4<T>(dk_row + 32 * nd + 8 * g + 4 * h, dk_t[nd], g, scale);
                    store4<T>(dv_row + 32 * nd + 8 * g + 4 * h, dv_t[nd], g, 1.0f);
                }
        }
    }
}

template <typename T, int DH, int MAX_TILES>
int launch_sized(const void* q, const void* k, const void* v, const void* g, void* dq, void* dk, void* dv, int B,
                 int H, int T_len, int P, float scale, int causal, hipStream_t stream) {
    constexpr size_t lds = lds_bytes<DH, MAX_TILES>();
    const int n_bh = B * H;
    const dim3 grid(grid_size(P, n_bh));
    auto run = [&](auto kern) {
        hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream, static_cast<const T*>(q), static_cast<const T*>(k),
                           static_cast<const T*>(v), static_cast<const T*>(g), static_cast<T*>(dq), static_cast<T*>(dk),
                           static_cast<T*>(dv), n_bh, H, P, T_len, scale);
    };
    if (causal) {
        if (int rc = ensure_dynamic_lds<&small_seq_kernel<T, DH, MAX_TILES, true>>(lds)) return rc;
        run(small_seq_kernel<T, DH, MAX_TILES, true>);
    } else {
        if (int rc = ensure_dynamic_lds<&small_seq_kernel<T, DH, MAX_TILES, false>>(lds)) return rc;
        run(small_seq_kernel<T, DH, MAX_TILES, false>);
    }
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

// T_len, dh as accepted by supports().
template <typename T>
int launch(const void* q, const void* k, const void* v, const void* g, void* dq, void* dk, void* dv, int B, int H,
           int T_len, int dh, int P, float scale, int causal, hipStream_t stream) {
    if (dh == 128) return launch_sized<T, 128, 4>(q, k, v, g, dq, dk, dv, B, H, T_len, P, scale, causal, stream);
    if (T_len <= 128) return launch_sized<T, 64, 4>(q, k, v, g, dq, dk, dv, B, H, T_len, P, scale, causal, stream);
    return launch_sized<T, 64, 8>(q, k, v, g, dq, dk, dv, B, H, T_len, P, scale, causal, stream);
}

}  // namespace attn_small
}  // namespace lbi
