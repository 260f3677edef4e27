// Attention input-pullback, MFMA path: fp16 / bf16 storage, head dim 64 or 128,
// T a multiple of 64, causal or not, fp32 accumulation.  (Short sequences run as one launch
// instead: lbi_attn_small.h, built from the same fragments.)
//
// Three kernels per call, all atomic-free (every output tile has one owner, sums run
// in a fixed order, so reruns are bit-identical):
//   stats_kernel  flash-style forward: lse2[b,h,i] (log2 domain) and O = softmax(..) V (fp32)
//   dq_ring_kernel    owner = 32 queries per wave, PB directions at once; streams K/V tiles
//                     (lbi_attn_dq128.h); it also forms -delta[b,p,h,i] = -sum_d d_out[b,p,h,i,d] * O[b,h,i,d]
//                     from the d_out tiles it holds anyway and leaves it in the workspace
//   dkdv_ring_kernel  owner = 64 keys per wave, one direction; streams Q/d_out tiles
//                     (lbi_attn_dkdv128.h)
//
// All products use v_mfma_f32_32x32x16_{bf16,f16}.  Operand layout (lane = 32*h + m):
//   A (32 x 16): lane holds A[m][8h .. 8h+7]     B (16 x 32): lane holds B[8h .. 8h+7][m]
//   C (32 x 32): register r of the lane holds C[row(r)][m],  row(r) = 8*(r/4) + 4*h + r%4
// Both inputs are "8 consecutive k per lane", so a row-major [rows][k] tile feeds either
// side with one 16-byte LDS read per lane ("nat" fragment).  When the reduction index is
// the ROW index of the tile in memory (d_out and Q in dK/dV, K in dQ, V in the forward),
// the fragment comes from the same tile through ds_read_b64_tr_b16 ("tr" fragment), which
// transposes 4x4 blocks of 16-bit elements across each group of 16 lanes.
//
// An accumulator tile C feeds the next product directly as its A or B operand, with the
// 32 rows of C as the reduction index: registers 8kk..8kk+7 are k-step kk and hold rows
// 16kk + {4h..4h+3, 8+4h..8+4h+3}; the tr fragment of the other operand is read with the
// same row assignment, so no data passes through LDS between the two products.
#pragma once

#include "lbi_common.h"

namespace lbi {
namespace attn_mfma {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr float LOG2E = 1.4426950408889634f;

// Scheduling fence between the phases of a tile step: keeps the compiler from
// interleaving phases, which only lengthens live ranges in these register-bound loops.
#ifndef LBI_ATTN_FENCE
#define LBI_ATTN_FENCE 1
#endif
#if LBI_ATTN_FENCE
#define LBI_PHASE_FENCE() __builtin_amdgcn_sched_barrier(0)
#else
#define LBI_PHASE_FENCE() ((void)0)
#endif

template <typename T> struct Mma;
template <> struct Mma<bf16_raw> {
    // Same product with the 32 x 32 result tile in ordinary VGPRs ("vgprcd" form).  The
    // compiler puts every builtin MFMA result in the 256 accumulation registers; a kernel
    // whose long-lived accumulators already fill those needs its short-lived S / dP tiles
    // elsewhere, or it shuffles registers on every step.  start(): C = 0.
    static __device__ __forceinline__ f32x16 mma_v_start(u32x4 a, u32x4 b) {
        f32x16 d;
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
        return d;
    }
    static __device__ __forceinline__ void mma_v(u32x4 a, u32x4 b, f32x16& c) {
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
    // start with C taken from another register tile (left untouched)
    static __device__ __forceinline__ f32x16 mma_v_c(u32x4 a, u32x4 b, const f32x16& c) {
        f32x16 d;
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
        return d;
    }
    static __device__ __forceinline__ float lo(unsigned w) { return __uint_as_float(w << 16); }
    static __device__ __forceinline__ float hi(unsigned w) { return __uint_as_float(w & 0xffff0000u); }
    static __device__ __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                       0, 0, 0);
    }
    static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
        // one v_cvt_pk_bf16_f32 (round to nearest even)
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
    }
};
template <> struct Mma<_Float16> {
    static __device__ __forceinline__ f32x16 mma_v_start(u32x4 a, u32x4 b) {
        f32x16 d;
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
        return d;
    }
    static __device__ __forceinline__ void mma_v(u32x4 a, u32x4 b, f32x16& c) {
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ f32x16 mma_v_c(u32x4 a, u32x4 b, const f32x16& c) {
        f32x16 d;
        asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "v"(a), "v"(b), "v"(c));
        return d;
    }
    static __device__ __forceinline__ float lo(unsigned w) { return (float)__builtin_bit_cast(f16x2, w)[0]; }
    static __device__ __forceinline__ float hi(unsigned w) { return (float)__builtin_bit_cast(f16x2, w)[1]; }
    static __device__ __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                      0, 0);
    }
    static __device__ __forceinline__ unsigned pack2(float lo, float hi) {
        const f32x2 v = {lo, hi};
        return __builtin_bit_cast(unsigned, __builtin_convertvector(v, f16x2));
    }
};

// Row of the 32 x 32 accumulator tile held in register r by a lane of half h.
__device__ __forceinline__ int c_row(int r, int h) { return 8 * (r >> 2) + 4 * h + (r & 3); }

// ---- LDS tiles: [32 rows][DH] 16-bit elements, 16-byte chunks XOR-swizzled so that both
// the nat reads (16 lanes = 16 rows, one chunk column) and the tr reads (4 rows x 64
// bytes per 32 lanes) touch every bank once.
template <int DH> __device__ __forceinline__ int swz(int r) {
    if (DH == 128) return ((r & 3) << 2) | ((r >> 2) & 3);
    const int x = r >> 1;  // DH == 64: two rows share one 256-byte bank line
    return ((x & 1) << 2) | ((x >> 1) & 3);
}
template <int DH> __device__ __forceinline__ int tile_off(int r, int chunk) {
    return r * (DH * 2) + ((chunk ^ swz<DH>(r)) << 4);
}

template <int DH> struct TileLoader {
    static constexpr int CHUNKS_PER_ROW = DH / 8;
    static constexpr int N = 32 * CHUNKS_PER_ROW / 256;  // 16-byte chunks per thread
    u32x4 regs[N];
    // rows row0 .. row0+31 of a row-major [T][DH] 16-bit matrix
    __device__ __forceinline__ void fetch(const void* base, int row0, int tid) {
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const int id = tid + 256 * u;
            const int r = id / CHUNKS_PER_ROW, c = id % CHUNKS_PER_ROW;
            regs[u] = *reinterpret_cast<const u32x4*>(static_cast<const char*>(base) +
                                                      ((size_t)(row0 + r) * DH + c * 8) * 2);
        }
    }
    __device__ __forceinline__ void commit(char* tile, int tid) const {
#pragma unroll
        for (int u = 0; u < N; ++u) {
            const int id = tid + 256 * u;
            const int r = id / CHUNKS_PER_ROW, c = id % CHUNKS_PER_ROW;
            *reinterpret_cast<u32x4*>(tile + tile_off<DH>(r, c)) = regs[u];
        }
    }
};

// nat fragment: lane (m, h) gets tile[m][16ks + 8h .. +7]
template <int DH> __device__ __forceinline__ u32x4 frag_nat(const char* tile, int m, int h, int ks) {
    return *reinterpret_cast<const u32x4*>(tile + tile_off<DH>(m, 2 * ks + h));
}

// tr fragment: lane (m, h) gets tile[k0 + {4h..4h+3, 8+4h..8+4h+3}][n0 + m]
template <int DH> __device__ __forceinline__ u32x4 frag_tr(const char* tile, int lane, int k0, int n0) {
    const int s = lane & 15, g1 = (lane >> 4) & 1, h = lane >> 5;
    const int row = k0 + 4 * h + (s >> 2);
    const int chunk = (n0 >> 3) + 2 * g1 + ((s & 3) >> 1);
    const int sub = (s & 1) << 3;
    typedef __attribute__((address_space(3))) s16x4* lds_ptr;
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + tile_off<DH>(row, chunk) + sub));
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + tile_off<DH>(row + 8, chunk) + sub));
    const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
    return u32x4{l2[0], l2[1], h2[0], h2[1]};
}

// Registers 8kk .. 8kk+7 of an accumulator tile as a 16-bit operand fragment.
template <typename T> __device__ __forceinline__ u32x4 pack_frag(const f32x16& c, int kk) {
    return u32x4{Mma<T>::pack2(c[8 * kk + 0], c[8 * kk + 1]), Mma<T>::pack2(c[8 * kk + 2], c[8 * kk + 3]),
                 Mma<T>::pack2(c[8 * kk + 4], c[8 * kk + 5]), Mma<T>::pack2(c[8 * kk + 6], c[8 * kk + 7])};
}

// The matrix pipe hands a VGPR-form result to the vector ALU only some cycles after issue,
// and nothing stalls an early reader.  The compiler pads its own MFMAs; after the ones
// issued through Mma<T>::mma_v the padding is explicit: 16 idle issue slots cover the
// 8-pass products used here.
__device__ __forceinline__ void mma_v_settle(f32x16& c0, f32x16& c1) {
    asm volatile("s_nop 15" : "+v"(c0), "+v"(c1));
}
__device__ __forceinline__ void mma_v_settle(f32x16& c0) { asm volatile("s_nop 15" : "+v"(c0)); }

// Pins the instructions that produce w0, w1 before this point in program order (the asm
// MFMAs are volatile too, so VALU work written between two of them stays between them
// and runs while the matrix pipe is busy).
__device__ __forceinline__ void pin_here(unsigned& w0, unsigned& w1) { asm volatile("" : "+v"(w0), "+v"(w1)); }

// Makes every later read of the tile depend on this point of the program (no instruction
// is emitted): work on the tile cannot be hoisted above it.
__device__ __forceinline__ void pin_tile(f32x16& c) { asm volatile("" : "+v"(c)); }

__device__ __forceinline__ f32x16 zero16() {
    f32x16 z;
#pragma unroll
    for (int e = 0; e < 16; ++e) z[e] = 0.0f;
    return z;
}

// Workgroup -> (b*H + h, rest): all workgroups of one (b, h) get ids that are equal
// mod 8, i.e. land on one XCD and share its L2 for that head's Q/K/V.
__device__ __forceinline__ bool map_block(int per_bh, int n_bh, int& bh, int& rem) {
    const int id = blockIdx.x;
    const int slot = id >> 3;
    bh = (slot / per_bh) * 8 + (id & 7);
    rem = slot % per_bh;
    return bh < n_bh;
}
inline unsigned grid_size(int per_bh, int n_bh) { return (unsigned)(((n_bh + 7) / 8) * 8 * per_bh); }

// ---------------------------------------------------------------------------------------
// stats_kernel: one wave = 32 queries, workgroup = 128 queries, K/V streamed in 32-key tiles.
// S^T tile: lanes = queries, registers = keys, so softmax statistics are per lane.
// ---------------------------------------------------------------------------------------
template <typename T, int DH, bool CAUSAL>
__global__ __launch_bounds__(256) void stats_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                    const T* __restrict__ v, float* __restrict__ lse2,
                                                    float* __restrict__ o32, int n_bh, int T_len, float scale) {
    constexpr int KS = DH / 16, ND = DH / 32, TILE_BYTES = 32 * DH * 2;
    extern __shared__ __align__(16) char smem[];  // [2][K tile, V tile]
    int bh, qb;
    const int n_qb = (T_len + 127) / 128;
    if (!map_block(n_qb, n_bh, bh, qb)) return;
    qb = n_qb - 1 - qb;  // longest rows first
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, m = lane & 31, h = lane >> 5;
    // Waves past the end of the sequence redo the last 32 rows and store nothing; the
    // loop body is branch-free so the accumulators stay in place.
    const bool active = qb * 128 + wave * 32 < T_len;
    const int i0w = min(qb * 128 + wave * 32, T_len - 32);
    const size_t base = (size_t)bh * T_len * DH;
    const T* k_bh = k + base;
    const T* v_bh = v + base;

    u32x4 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        qf[ks] = *reinterpret_cast<const u32x4*>(q + base + (size_t)(i0w + m) * DH + 16 * ks + 8 * h);
    f32x16 o_t[ND];
#pragma unroll
    for (int nd = 0; nd < ND; ++nd) o_t[nd] = zero16();
    float m_run = -INFINITY, l_run = 0.0f;
    const float sc2 = scale * LOG2E;

    const int j_end = CAUSAL ? min(T_len, qb * 128 + 128) : T_len;
    const int n_it = j_end / 32;
    TileLoader<DH> kl, vl;
    kl.fetch(k_bh, 0, tid);
    vl.fetch(v_bh, 0, tid);
    kl.commit(smem, tid);
    vl.commit(smem + TILE_BYTES, tid);
    __syncthreads();
    for (int it = 0; it < n_it; ++it) {
        const int j0 = it * 32;
        const char* kt = smem + (it & 1) * 2 * TILE_BYTES;
        const char* vt = kt + TILE_BYTES;
        {
            const int j_next = min(j0 + 32, T_len - 32);  // the last trip re-reads a valid tile
            kl.fetch(k_bh, j_next, tid);
            vl.fetch(v_bh, j_next, tid);
        }
        {
            // A tile that lies wholly above the diagonal masks to all -inf and changes nothing.
            f32x16 s = zero16();
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) s = Mma<T>::mma(frag_nat<DH>(kt, m, h, ks), qf[ks], s);
            const bool diag = CAUSAL && (j0 + 31 > i0w);
            float tmax = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float x = s[r] * sc2;
                if (diag && (j0 + c_row(r, h) > i0w + m)) x = -INFINITY;
                s[r] = x;
                tmax = fmaxf(tmax, x);
            }
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
            // The reference point of the exponentials follows the running maximum only when that has grown by
            // more than 2^8 (or is seen for the first time): the sums then carry terms of up to 2^8 instead of
            // 1, which fp32 does not notice, and the rescaling of the 64 accumulator values of a lane, otherwise
            // due on most steps, happens a few times per row.  O / l and m + log2 l do not depend on the choice.
            const float m_new = fmaxf(m_run, tmax);
            const bool grow = (m_run == -INFINITY) ? (m_new != -INFINITY) : (m_new - m_run > 8.0f);
            const float m_use = grow ? m_new : m_run;
            float lsum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pr = (m_use == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(s[r] - m_use);
                s[r] = pr;
                lsum += pr;
            }
            lsum += __shfl_xor(lsum, 32, 64);
            if (__builtin_amdgcn_ballot_w64(grow) != 0) {  // wave-uniform
                const float alpha = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run - m_use);
                l_run *= alpha;
#pragma unroll
                for (int nd = 0; nd < ND; ++nd)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o_t[nd][r] *= alpha;
            }
            l_run += lsum;
            m_run = m_use;
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) {
                const u32x4 pb = pack_frag<T>(s, kk);
#pragma unroll
                for (int nd = 0; nd < ND; ++nd)
                    o_t[nd] = Mma<T>::mma(frag_tr<DH>(vt, lane, 16 * kk, 32 * nd), pb, o_t[nd]);
            }
        }
        {
            char* nxt = smem + ((it + 1) & 1) * 2 * TILE_BYTES;
            kl.commit(nxt, tid);
            vl.commit(nxt + TILE_BYTES, tid);
        }
        __syncthreads();
    }
    if (active) {
        const float inv = 1.0f / l_run;
        if (h == 0) lse2[(size_t)bh * T_len + i0w + m] = m_run + log2f(l_run);
        float* o_row = o32 + base + (size_t)(i0w + m) * DH;
#pragma unroll
        for (int nd = 0; nd < ND; ++nd)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                f32x4 o4 = {o_t[nd][4 * g] * inv, o_t[nd][4 * g + 1] * inv, o_t[nd][4 * g + 2] * inv,
                            o_t[nd][4 * g + 3] * inv};
                *reinterpret_cast<f32x4*>(o_row + 32 * nd + 8 * g + 4 * h) = o4;
            }
    }
}

inline bool supports(int T_len, int dh, int dtype) {
    return (dtype == LBI_F16 || dtype == LBI_BF16) && (dh == 64 || dh == 128) && T_len >= 64 && T_len % 64 == 0;
}

// floats: lse2[B*H*T], -delta[B*P*H*T], o32[B*H*T*Dh]
inline size_t workspace_floats(int64_t B, int64_t H, int64_t T, int64_t Dh, int64_t P) {
    return (size_t)(B * H * T + B * P * H * T + B * H * T * Dh);
}

// dK/dV launch (kernel in lbi_attn_dkdv128.h).
template <typename T, int DH, bool CAUSAL>
int launch_dkdv(const T* q, const T* k, const T* v, const T* g, const float* lse2, const float* delta, T* dk, T* dv,
                 int n_bh, int H, int P, int T_len, float scale, hipStream_t stream);

// dK/dV launch for two or more directions (kernel in lbi_attn_dkdv_pair.h).
template <typename T, int DH, bool CAUSAL>
int launch_dkdv_pair(const T* q, const T* k, const T* v, const T* g, const float* lse2, const float* delta, T* dk,
                      T* dv, int n_bh, int H, int P, int T_len, float scale, hipStream_t stream);

// dQ launch (kernel in lbi_attn_dq128.h); PB = directions per wave.
template <typename T, int DH, int PB, bool CAUSAL>
int launch_dq(const T* q, const T* k, const T* v, const T* g, const float* lse2, const float* o32, float* delta, T* dq,
               int n_bh, int H, int P, int T_len, float scale, hipStream_t stream);

template <typename T, int DH, bool CAUSAL>
int launch_typed(const T* q, const T* k, const T* v, const T* g, T* dq, T* dk, T* dv, float* workspace, int B,
                 int H, int T_len, int P, float scale, hipStream_t stream) {
    constexpr size_t lds_bytes = 4 * 32 * DH * 2;
    const int n_bh = B * H;
    float* lse2 = workspace;
    float* delta = lse2 + (size_t)n_bh * T_len;
    float* o32 = delta + (size_t)n_bh * P * T_len;
    const int n_qb = (T_len + 127) / 128;
    hipLaunchKernelGGL((stats_kernel<T, DH, CAUSAL>), dim3(grid_size(n_qb, n_bh)), dim3(256), lds_bytes, stream, q, k,
                       v, lse2, o32, n_bh, T_len, scale);
    // the dQ kernel runs first: it writes -delta, which the dK/dV kernel reads
    // directions per wave of the dQ kernel: as many as share one S tile, without idle slots for one or two directions
    int rc;
    if (P == 1) rc = launch_dq<T, DH, 1, CAUSAL>(q, k, v, g, lse2, o32, delta, dq, n_bh, H, P, T_len, scale, stream);
    else if (P == 2) rc = launch_dq<T, DH, 2, CAUSAL>(q, k, v, g, lse2, o32, delta, dq, n_bh, H, P, T_len, scale, stream);
    else if (DH == 64 && P > 4) rc = launch_dq<T, DH, 8, CAUSAL>(q, k, v, g, lse2, o32, delta, dq, n_bh, H, P, T_len, scale, stream);
    else rc = launch_dq<T, DH, 4, CAUSAL>(q, k, v, g, lse2, o32, delta, dq, n_bh, H, P, T_len, scale, stream);
    if (rc) return rc;
    if (P >= 2) rc = launch_dkdv_pair<T, DH, CAUSAL>(q, k, v, g, lse2, delta, dk, dv, n_bh, H, P, T_len, scale, stream);
    else rc = launch_dkdv<T, DH, CAUSAL>(q, k, v, g, lse2, delta, dk, dv, n_bh, H, P, T_len, scale, stream);
    if (rc) return rc;
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

template <typename T>
int launch(const void* q, const void* k, const void* v, const void* g, void* dq, void* dk, void* dv, float* workspace,
           int B, int H, int T_len, int dh, int P, float scale, int causal, hipStream_t stream) {
    const T* qp = static_cast<const T*>(q);
    const T* kp = static_cast<const T*>(k);
    const T* vp = static_cast<const T*>(v);
    const T* gp = static_cast<const T*>(g);
    T* dqp = static_cast<T*>(dq);
    T* dkp = static_cast<T*>(dk);
    T* dvp = static_cast<T*>(dv);
    if (dh == 128) {
        return causal ? launch_typed<T, 128, true>(qp, kp, vp, gp, dqp, dkp, dvp, workspace, B, H, T_len, P, scale, stream)
                      : launch_typed<T, 128, false>(qp, kp, vp, gp, dqp, dkp, dvp, workspace, B, H, T_len, P, scale, stream);
    }
    return causal ? launch_typed<T, 64, true>(qp, kp, vp, gp, dqp, dkp, dvp, workspace, B, H, T_len, P, scale, stream)
                  : launch_typed<T, 64, false>(qp, kp, vp, gp, dqp, dkp, dvp, workspace, B, H, T_len, P, scale, stream);
}

}  // namespace attn_mfma
}  // namespace lbi
