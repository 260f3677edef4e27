// Attention input-pullback, MFMA path: fp16 / bf16 storage, head dim 64 or 128,
// T a multiple of 64, causal or not, fp32 accumulation.
//
// Four kernels per call, all atomic-free (every output tile has one owner, sums run
// in a fixed order, so reruns are bit-identical):
//   stats_kernel  flash-style forward: lse2[b,h,i] (log2 domain) and O = softmax(..) V (fp32)
//   delta_kernel  delta[b,p,h,i] = sum_d d_out[b,p,h,i,d] * O[b,h,i,d]
//   dq_kernel     owner = 32 queries per wave, PB directions at once; streams K/V tiles
//   dkdv_kernel   owner = 64 keys per wave, one direction; streams Q/d_out tiles
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
            const float m_new = fmaxf(m_run, tmax);
            const float alpha = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(m_run - m_new);
            float lsum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float pr = (m_new == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f(s[r] - m_new);
                s[r] = pr;
                lsum += pr;
            }
            lsum += __shfl_xor(lsum, 32, 64);
            l_run = l_run * alpha + lsum;
            m_run = m_new;
#pragma unroll
            for (int nd = 0; nd < ND; ++nd)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_t[nd][r] *= alpha;
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

// ---------------------------------------------------------------------------------------
// delta_kernel: DH/8 lanes per row, 16 bytes of d_out and 32 bytes of O per lane.
// ---------------------------------------------------------------------------------------
template <typename T, int DH>
__global__ __launch_bounds__(256) void delta_kernel(const T* __restrict__ d_out, const float* __restrict__ o32,
                                                    float* __restrict__ delta, int H, int P, int T_len,
                                                    size_t n_rows) {
    constexpr int LPR = DH / 8;  // lanes per row
    const size_t row = (size_t)blockIdx.x * (256 / LPR) + threadIdx.x / LPR;
    const int part = threadIdx.x % LPR;
    float acc = 0.0f;
    if (row < n_rows) {
        const size_t t = row % T_len;
        const size_t bph = row / T_len;
        const size_t h = bph % H, b = bph / ((size_t)H * P);
        const size_t o_row = (b * H + h) * T_len + t;
        const u32x4 g = *reinterpret_cast<const u32x4*>(d_out + row * DH + part * 8);
        const f32x4 o_lo = *reinterpret_cast<const f32x4*>(o32 + o_row * DH + part * 8);
        const f32x4 o_hi = *reinterpret_cast<const f32x4*>(o32 + o_row * DH + part * 8 + 4);
        const T* ge = reinterpret_cast<const T*>(&g);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = fmaf(to_f32(ge[e]), o_lo[e], acc);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = fmaf(to_f32(ge[4 + e]), o_hi[e], acc);
    }
#pragma unroll
    for (int off = LPR / 2; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, LPR);
    if (part == 0 && row < n_rows) delta[row] = acc;
}

// ---------------------------------------------------------------------------------------
// dq_kernel: one wave = 32 queries x PB directions; Q and the PB d_out tiles of those
// queries stay in registers as B operands; K/V stream through LDS in 32-key tiles.
//   S^T  = K Q^T      (A = K nat, B = Q)         lanes = queries, registers = keys
//   dP^T = V dO_p^T   (A = V nat, B = dO_p)
//   dQ_p += dS_p K    (A = dS_p from registers, B = K tr)   lanes = d, registers = queries
// ---------------------------------------------------------------------------------------
template <typename T, int DH, int PB, bool CAUSAL>
__global__ __launch_bounds__(256) void dq_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                 const T* __restrict__ v, const T* __restrict__ d_out,
                                                 const float* __restrict__ lse2, const float* __restrict__ delta,
                                                 T* __restrict__ dq, int n_bh, int H, int P, int T_len,
                                                 float scale) {
    constexpr int KS = DH / 16, ND = DH / 32, TILE_BYTES = 32 * DH * 2;
    extern __shared__ __align__(16) char smem[];  // [2][K tile, V tile]
    const int n_qb = (T_len + 127) / 128;
    const int n_pb = (P + PB - 1) / PB;
    int bh, rem;
    if (!map_block(n_qb * n_pb, n_bh, bh, rem)) return;
    const int qb = n_qb - 1 - rem / n_pb;  // longest rows first
    const int p0 = (rem % n_pb) * PB;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, m = lane & 31, h = lane >> 5;
    const bool active = qb * 128 + wave * 32 < T_len;
    const int i0w = min(qb * 128 + wave * 32, T_len - 32);  // see stats_kernel
    const size_t base = (size_t)bh * T_len * DH;
    const T* k_bh = k + base;
    const T* v_bh = v + base;

    u32x4 qf[KS], gf[PB][KS];
    float my_delta[PB];
    float my_lse = 0.0f;
    {
        my_lse = lse2[(size_t)bh * T_len + i0w + m];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            qf[ks] = *reinterpret_cast<const u32x4*>(q + base + (size_t)(i0w + m) * DH + 16 * ks + 8 * h);
#pragma unroll
        for (int pp = 0; pp < PB; ++pp) {
            const int p = min(p0 + pp, P - 1);  // surplus slots recompute the last direction; never stored
            const size_t row = (((size_t)b * P + p) * H + hh) * T_len + i0w + m;
            my_delta[pp] = delta[row];
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                gf[pp][ks] = *reinterpret_cast<const u32x4*>(d_out + row * DH + 16 * ks + 8 * h);
        }
    }
    f32x16 acc[PB][ND];
#pragma unroll
    for (int pp = 0; pp < PB; ++pp)
#pragma unroll
        for (int nd = 0; nd < ND; ++nd) acc[pp][nd] = zero16();
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
            const int j_next = min(j0 + 32, T_len - 32);
            kl.fetch(k_bh, j_next, tid);
            vl.fetch(v_bh, j_next, tid);
        }
        {
            // A tile wholly above the diagonal gets P = 0 and adds nothing.
            f32x16 s = zero16();
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) s = Mma<T>::mma(frag_nat<DH>(kt, m, h, ks), qf[ks], s);
            const bool diag = CAUSAL && (j0 + 31 > i0w);
            u32x4 pq[2];  // P rounded to the storage type (see dkdv_kernel)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float pr[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    pr[e] = __builtin_amdgcn_exp2f(s[4 * g + e] * sc2 - my_lse);
                    if (diag && (j0 + 8 * g + 4 * h + e > i0w + m)) pr[e] = 0.0f;
                }
                pq[g >> 1][2 * (g & 1)] = Mma<T>::pack2(pr[0], pr[1]);
                pq[g >> 1][2 * (g & 1) + 1] = Mma<T>::pack2(pr[2], pr[3]);
            }
            LBI_PHASE_FENCE();
            f32x16 dp[PB];
#pragma unroll
            for (int pp = 0; pp < PB; ++pp) dp[pp] = zero16();
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const u32x4 vfrag = frag_nat<DH>(vt, m, h, ks);
#pragma unroll
                for (int pp = 0; pp < PB; ++pp) dp[pp] = Mma<T>::mma(vfrag, gf[pp][ks], dp[pp]);
            }
            u32x4 dsa[PB][2];
#pragma unroll
            for (int pp = 0; pp < PB; ++pp)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const unsigned w0 = pq[g >> 1][2 * (g & 1)], w1 = pq[g >> 1][2 * (g & 1) + 1];
                    const float d0 = Mma<T>::lo(w0) * (dp[pp][4 * g + 0] - my_delta[pp]);
                    const float d1 = Mma<T>::hi(w0) * (dp[pp][4 * g + 1] - my_delta[pp]);
                    const float d2 = Mma<T>::lo(w1) * (dp[pp][4 * g + 2] - my_delta[pp]);
                    const float d3 = Mma<T>::hi(w1) * (dp[pp][4 * g + 3] - my_delta[pp]);
                    dsa[pp][g >> 1][2 * (g & 1)] = Mma<T>::pack2(d0, d1);
                    dsa[pp][g >> 1][2 * (g & 1) + 1] = Mma<T>::pack2(d2, d3);
                }
            LBI_PHASE_FENCE();
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
#pragma unroll
                for (int nd = 0; nd < ND; ++nd) {
                    const u32x4 kfrag = frag_tr<DH>(kt, lane, 16 * kk, 32 * nd);
#pragma unroll
                    for (int pp = 0; pp < PB; ++pp) acc[pp][nd] = Mma<T>::mma(dsa[pp][kk], kfrag, acc[pp][nd]);
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
#pragma unroll
        for (int pp = 0; pp < PB; ++pp) {
            if (p0 + pp >= P) break;
            T* out = dq + ((((size_t)b * P + p0 + pp) * H + hh) * T_len + i0w) * DH;
#pragma unroll
            for (int nd = 0; nd < ND; ++nd)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    // rows r and r+1 of this lane's column; one 16-bit store each
                    const unsigned two = Mma<T>::pack2(acc[pp][nd][r] * scale, acc[pp][nd][r + 1] * scale);
                    unsigned short* o = reinterpret_cast<unsigned short*>(out);
                    o[(size_t)c_row(r, h) * DH + 32 * nd + m] = (unsigned short)(two & 0xffffu);
                    o[(size_t)c_row(r + 1, h) * DH + 32 * nd + m] = (unsigned short)(two >> 16);
                }
        }
    }
}

// ---------------------------------------------------------------------------------------
// dkdv_kernel: one wave = 64 keys x one direction, workgroup = 256 keys; K and V of those
// keys stay in registers as B operands; Q and d_out_p stream through LDS in 32-query tiles.
//   S    = Q K^T      (A = Q nat,    B = K)      lanes = keys, registers = queries
//   dP   = dO_p V^T   (A = dO_p nat, B = V)
//   dV_p += P^T dO_p  (A = P from registers,    B = dO_p tr)   lanes = d, registers = keys
//   dK_p += dS^T Q    (A = dS_p from registers, B = Q tr)
// ---------------------------------------------------------------------------------------
template <typename T, int DH, bool CAUSAL>
__global__ __launch_bounds__(256) void dkdv_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                   const T* __restrict__ v, const T* __restrict__ d_out,
                                                   const float* __restrict__ lse2, const float* __restrict__ delta,
                                                   T* __restrict__ dk, T* __restrict__ dv, int n_bh, int H, int P,
                                                   int T_len, float scale) {
    constexpr int KS = DH / 16, ND = DH / 32, TILE_BYTES = 32 * DH * 2;
    extern __shared__ __align__(16) char smem[];  // [2][Q tile, dO tile]
    const int n_kb = (T_len + 255) / 256;
    int bh, rem;
    if (!map_block(n_kb * P, n_bh, bh, rem)) return;
    const int p = rem / n_kb;
    const int kb = rem % n_kb;  // key block 0 sees the most queries and starts first
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, m = lane & 31, h = lane >> 5;
    const bool active = kb * 256 + wave * 64 < T_len;
    const int j0w = min(kb * 256 + wave * 64, T_len - 64);  // see stats_kernel
    const size_t base = (size_t)bh * T_len * DH;
    const size_t prow = (((size_t)b * P + p) * H + hh) * T_len;
    const T* q_bh = q + base;
    const T* g_p = d_out + prow * DH;
    const float* lse_bh = lse2 + (size_t)bh * T_len;
    const float* delta_p = delta + prow;

    u32x4 kf[2][KS], vf[2][KS];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const size_t off = base + (size_t)(j0w + 32 * t + m) * DH + 16 * ks + 8 * h;
            kf[t][ks] = *reinterpret_cast<const u32x4*>(k + off);
            vf[t][ks] = *reinterpret_cast<const u32x4*>(v + off);
        }
    f32x16 acc_k[2][ND], acc_v[2][ND];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int nd = 0; nd < ND; ++nd) {
            acc_k[t][nd] = zero16();
            acc_v[t][nd] = zero16();
        }
    const float sc2 = scale * LOG2E;

    const int i_begin = CAUSAL ? kb * 256 : 0;
    const int n_it = (T_len - i_begin) / 32;
    // The 32 lse2 and 32 delta values of a query tile travel with it through LDS
    // (threads 0-7 carry lse2, 8-15 delta, one float4 each).
    float* row_stats = reinterpret_cast<float*>(smem + 4 * TILE_BYTES);  // [2][64]
    const float* stat_src = (tid < 8 ? lse_bh : delta_p) + 4 * (tid & 7);
    f32x4 stat_reg = {0.0f, 0.0f, 0.0f, 0.0f};
    TileLoader<DH> ql, gl;
    ql.fetch(q_bh, i_begin, tid);
    gl.fetch(g_p, i_begin, tid);
    if (tid < 16) stat_reg = *reinterpret_cast<const f32x4*>(stat_src + i_begin);
    ql.commit(smem, tid);
    gl.commit(smem + TILE_BYTES, tid);
    if (tid < 16) *reinterpret_cast<f32x4*>(row_stats + 4 * tid) = stat_reg;
    __syncthreads();
    for (int it = 0; it < n_it; ++it) {
        const int i0 = i_begin + it * 32;
        const char* qt = smem + (it & 1) * 2 * TILE_BYTES;
        const char* gt = qt + TILE_BYTES;
        const float* lse_t = row_stats + (it & 1) * 64;
        const float* delta_t = lse_t + 32;
        {
            const int i_next = min(i0 + 32, T_len - 32);
            ql.fetch(q_bh, i_next, tid);
            gl.fetch(g_p, i_next, tid);
            if (tid < 16) stat_reg = *reinterpret_cast<const f32x4*>(stat_src + i_next);
        }
        {
            // Query tiles wholly before this wave's keys get P = 0 and add nothing.
            f32x16 s[2] = {zero16(), zero16()};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const u32x4 a = frag_nat<DH>(qt, m, h, ks);
                s[0] = Mma<T>::mma(a, kf[0][ks], s[0]);
                s[1] = Mma<T>::mma(a, kf[1][ks], s[1]);
            }
            // P = exp2(S*c - lse2), rounded to the storage type at once: the rounded values
            // feed both dV and dS, and the fp32 tile dies here (register budget).
            const bool diag = CAUSAL && (j0w + 63 > i0);
            u32x4 pa[2][2], dsa[2][2];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 l4 = *reinterpret_cast<const f32x4*>(lse_t + 8 * g + 4 * h);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    float pr[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        pr[e] = __builtin_amdgcn_exp2f(s[t][4 * g + e] * sc2 - l4[e]);
                        if (diag && (j0w + 32 * t + m > i0 + 8 * g + 4 * h + e)) pr[e] = 0.0f;
                    }
                    pa[t][g >> 1][2 * (g & 1)] = Mma<T>::pack2(pr[0], pr[1]);
                    pa[t][g >> 1][2 * (g & 1) + 1] = Mma<T>::pack2(pr[2], pr[3]);
                }
            }
            LBI_PHASE_FENCE();
            f32x16 dp[2] = {zero16(), zero16()};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const u32x4 a = frag_nat<DH>(gt, m, h, ks);
                dp[0] = Mma<T>::mma(a, vf[0][ks], dp[0]);
                dp[1] = Mma<T>::mma(a, vf[1][ks], dp[1]);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const f32x4 d4 = *reinterpret_cast<const f32x4*>(delta_t + 8 * g + 4 * h);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const unsigned w0 = pa[t][g >> 1][2 * (g & 1)], w1 = pa[t][g >> 1][2 * (g & 1) + 1];
                    const float d0 = Mma<T>::lo(w0) * (dp[t][4 * g + 0] - d4[0]);
                    const float d1 = Mma<T>::hi(w0) * (dp[t][4 * g + 1] - d4[1]);
                    const float d2 = Mma<T>::lo(w1) * (dp[t][4 * g + 2] - d4[2]);
                    const float d3 = Mma<T>::hi(w1) * (dp[t][4 * g + 3] - d4[3]);
                    dsa[t][g >> 1][2 * (g & 1)] = Mma<T>::pack2(d0, d1);
                    dsa[t][g >> 1][2 * (g & 1) + 1] = Mma<T>::pack2(d2, d3);
                }
            }
            LBI_PHASE_FENCE();
            // tr fragments are fetched one (kk, nd) step ahead of the products that use them.
            u32x4 bg = frag_tr<DH>(gt, lane, 0, 0), bq = frag_tr<DH>(qt, lane, 0, 0);
#pragma unroll
            for (int step = 0; step < 2 * ND; ++step) {
                const int kk = step / ND, nd = step % ND;
                u32x4 bg_n = bg, bq_n = bq;
                if (step + 1 < 2 * ND) {
                    bg_n = frag_tr<DH>(gt, lane, 16 * ((step + 1) / ND), 32 * ((step + 1) % ND));
                    bq_n = frag_tr<DH>(qt, lane, 16 * ((step + 1) / ND), 32 * ((step + 1) % ND));
                }
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    acc_v[t][nd] = Mma<T>::mma(pa[t][kk], bg, acc_v[t][nd]);
                    acc_k[t][nd] = Mma<T>::mma(dsa[t][kk], bq, acc_k[t][nd]);
                }
                bg = bg_n;
                bq = bq_n;
                LBI_PHASE_FENCE();
            }
        }
        {
            char* nxt = smem + ((it + 1) & 1) * 2 * TILE_BYTES;
            ql.commit(nxt, tid);
            gl.commit(nxt + TILE_BYTES, tid);
            if (tid < 16) *reinterpret_cast<f32x4*>(row_stats + ((it + 1) & 1) * 64 + 4 * tid) = stat_reg;
        }
        __syncthreads();
    }
    if (active) {
        unsigned short* ok = reinterpret_cast<unsigned short*>(dk + (prow + j0w) * DH);
        unsigned short* ov = reinterpret_cast<unsigned short*>(dv + (prow + j0w) * DH);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int nd = 0; nd < ND; ++nd)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    const unsigned k2 = Mma<T>::pack2(acc_k[t][nd][r] * scale, acc_k[t][nd][r + 1] * scale);
                    const unsigned v2 = Mma<T>::pack2(acc_v[t][nd][r], acc_v[t][nd][r + 1]);
                    const size_t o0 = (size_t)(32 * t + c_row(r, h)) * DH + 32 * nd + m;
                    const size_t o1 = (size_t)(32 * t + c_row(r + 1, h)) * DH + 32 * nd + m;
                    ok[o0] = (unsigned short)(k2 & 0xffffu);
                    ok[o1] = (unsigned short)(k2 >> 16);
                    ov[o0] = (unsigned short)(v2 & 0xffffu);
                    ov[o1] = (unsigned short)(v2 >> 16);
                }
    }
}

inline bool supports(int T_len, int dh, int dtype) {
    return (dtype == LBI_F16 || dtype == LBI_BF16) && (dh == 64 || dh == 128) && T_len >= 64 && T_len % 64 == 0;
}

// floats: lse2[B*H*T], delta[B*P*H*T], o32[B*H*T*Dh]
inline size_t workspace_floats(int64_t B, int64_t H, int64_t T, int64_t Dh, int64_t P) {
    return (size_t)(B * H * T + B * P * H * T + B * H * T * Dh);
}

// dK/dV launch: head dim 128 has its own kernel (lbi_attn_dkdv128.h).
template <typename T, int DH, bool CAUSAL>
void launch_dkdv(const T* q, const T* k, const T* v, const T* g, const float* lse2, const float* delta, T* dk, T* dv,
                 int n_bh, int H, int P, int T_len, float scale, hipStream_t stream);

// dQ launch: head dim 128 has its own kernel (lbi_attn_dq128.h).
template <typename T, int DH, int PB, bool CAUSAL>
void launch_dq(const T* q, const T* k, const T* v, const T* g, const float* lse2, const float* delta, T* dq, int n_bh,
               int H, int P, int T_len, float scale, hipStream_t stream);

template <typename T, int DH, bool CAUSAL>
int launch_typed(const T* q, const T* k, const T* v, const T* g, T* dq, T* dk, T* dv, float* workspace, int B,
                 int H, int T_len, int P, float scale, hipStream_t stream) {
    constexpr int PB = DH == 128 ? 2 : 4;
    constexpr size_t lds_bytes = 4 * 32 * DH * 2;
    constexpr size_t lds_bytes_dkdv = lds_bytes + 2 * 64 * sizeof(float);
    const int n_bh = B * H;
    float* lse2 = workspace;
    float* delta = lse2 + (size_t)n_bh * T_len;
    float* o32 = delta + (size_t)n_bh * P * T_len;
    const int n_qb = (T_len + 127) / 128;
    const int n_kb = (T_len + 255) / 256;
    const int n_pb = (P + PB - 1) / PB;
    hipLaunchKernelGGL((stats_kernel<T, DH, CAUSAL>), dim3(grid_size(n_qb, n_bh)), dim3(256), lds_bytes, stream, q, k,
                       v, lse2, o32, n_bh, T_len, scale);
    const size_t n_rows = (size_t)n_bh * P * T_len;
    constexpr int rows_per_block = 256 / (DH / 8);
    hipLaunchKernelGGL((delta_kernel<T, DH>), dim3((unsigned)((n_rows + rows_per_block - 1) / rows_per_block)),
                       dim3(256), 0, stream, g, o32, delta, H, P, T_len, n_rows);
    launch_dq<T, DH, PB, CAUSAL>(q, k, v, g, lse2, delta, dq, n_bh, H, P, T_len, scale, stream);
    launch_dkdv<T, DH, CAUSAL>(q, k, v, g, lse2, delta, dk, dv, n_bh, H, P, T_len, scale, stream);
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
