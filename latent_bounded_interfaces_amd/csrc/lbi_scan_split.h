// Suffix scan for d = 256 on the 16-bit matrix pipes, with fp32-exact products.
//
// The fp32 MFMA rate of gfx950 is 1/16 of its bf16 rate, so the scan of d = 256 matrices
// is bound by the matrix pipes when its products run as fp32 MFMAs.  Here every fp32
// number x is split exactly into three bf16 numbers, x = hi + mid + lo (8 + 8 + 8
// significand bits, round-to-nearest residuals), so
//     a * s = sum over the planes of (a_i * s_j),   each a_i * s_j exact in fp32,
// and the products are v_mfma_f32_32x32x16_bf16 accumulated in fp32.  Nothing is dropped:
// bf16 storage (NA = 1, the matrix is one plane) costs 3 bf16 products per fp32 product,
// fp32 storage (NA = 3) costs 9, against 16 for one fp32 MFMA product.  The results differ
// from the fp32-MFMA kernel only in summation order; partial products are summed in two
// accumulators (hi*hi | everything smaller), small terms first.
//
// Layout is that of scan_mfma_kernel: a workgroup owns 64 columns of one batch element's
// running suffix S, streams mats[b, K-1 .. 0] once, one wave owns 32 rows.  S lives in LDS
// as three bf16 planes, transposed ([plane][col][k], pitch 264 elements: 16-byte reads of
// 16 lanes hit 64 distinct banks), single buffered (two barriers per step).  mats rows go
// global -> registers, 64 bytes per lane per chunk, through a 4-slot ring filled 3 chunks
// ahead across step boundaries.  COT: also run the cotangent chain (see scan_mfma_kernel).
#pragma once

#include "lbi_common.h"

// Plane pairs (a_i, s_j) with i + j above this are skipped.  4 keeps all nine products of two
// fp32 numbers (exact); 2 would drop terms of relative size 2^-24 and below.
#ifndef LBI_SPLIT_MAX_ORDER
#define LBI_SPLIT_MAX_ORDER 4
#endif

namespace lbi {
namespace scan_split {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int D = 256, CB = 64, RT = 32, NW = D / RT, NT = 64 * NW, NB = D / CB;
constexpr int PITCH = D + 8;              // bf16 elements per plane row
constexpr int PLANE = CB * PITCH;         // elements per plane
constexpr size_t PLANES_BYTES = (size_t)3 * PLANE * 2;

__device__ __forceinline__ unsigned pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));  // v_cvt_pk_bf16_f32, RNE
}
__device__ __forceinline__ float bf16_lo(unsigned w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(unsigned w) { return __uint_as_float(w & 0xffff0000u); }

// x0, x1 -> three packed words (hi, mid, lo planes); hi + mid + lo == x exactly.
__device__ __forceinline__ void split2(float x0, float x1, unsigned& hi, unsigned& mid, unsigned& lo) {
    hi = pack_bf16(x0, x1);
    const float r0 = x0 - bf16_lo(hi), r1 = x1 - bf16_hi(hi);
    mid = pack_bf16(r0, r1);
    lo = pack_bf16(r0 - bf16_lo(mid), r1 - bf16_hi(mid));
}

__device__ __forceinline__ f32x16 mma(u32x4 a, u32x4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0,
                                                   0);
}

// Raw chunk of a lane: 64 bytes of its row.
//   bf16 storage: 32 consecutive k  (chunk = 64 k: the h = 0 / 1 lanes take k 0-31 / 32-63), 4 products
//   fp32 storage: 16 consecutive k  (chunk = 32 k),                                         2 products
template <typename Tin> struct Chunk;
template <> struct Chunk<bf16_raw> {
    static constexpr int K_PER_CHUNK = 64, K_PER_LANE = 32, T_STEPS = 4, NA = 1;
};
template <> struct Chunk<float> {
    static constexpr int K_PER_CHUNK = 32, K_PER_LANE = 16, T_STEPS = 2, NA = 3;
};

// NP = planes of the running suffix that enter the products: 3 is exact; 2 (bf16 storage only) rounds that operand
// to 16 significand bits (hi + mid), accumulation and stored results stay fp32.
template <typename Tin, bool COT, int NP>
__global__ __launch_bounds__(NT) void scan_split_kernel(const Tin* __restrict__ mats, float* __restrict__ out,
                                                        const float* __restrict__ g, float* __restrict__ cot, int B,
                                                        int K) {
    using C = Chunk<Tin>;
    constexpr int NCH = D / C::K_PER_CHUNK;  // chunks per step: 4 (bf16) or 8 (fp32)
    constexpr int RING = 4, AHEAD = RING - 1;
    constexpr int NA = C::NA;
    static_assert(NCH % RING == 0, "ring slots must be compile-time constants");

    extern __shared__ __align__(16) char smem[];
    unsigned short* planes = reinterpret_cast<unsigned short*>(smem);        // [3][CB][PITCH]
    float* vbuf = reinterpret_cast<float*>(smem + (size_t)NP * PLANE * 2);  // (COT) [2][D], behind the NP planes

    const int id = blockIdx.x;
    const int slot_id = id >> 3;
    const int b = (slot_id / NB) * 8 + (id & 7);
    const int c0 = (slot_id % NB) * CB;
    if (b >= B) return;
    const int tid = threadIdx.x, lane = tid & 63, m = lane & 31, h = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int row0 = wave * RT;
    const Tin* mats_b = mats + (size_t)b * K * D * D;
    float* out_b = out + (size_t)b * (K + 1) * D * D;
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // Identity tail, first suffix (= mats[K-1]) and its planes.
    {
        const Tin* a_last = mats_b + (size_t)(K - 1) * D * D;
        float* o_last = out_b + (size_t)(K - 1) * D * D;
        float* o_eye = out_b + (size_t)K * D * D;
        for (int idx = tid; idx < D * CB; idx += NT) {
            const int row = idx / CB, col = idx % CB;
            const float val = to_f32(a_last[row * D + c0 + col]);
            o_last[row * D + c0 + col] = val;
            o_eye[row * D + c0 + col] = (row == c0 + col) ? 1.0f : 0.0f;
            unsigned hi, mid, lo;
            split2(val, 0.0f, hi, mid, lo);
            planes[0 * PLANE + col * PITCH + row] = (unsigned short)hi;
            planes[1 * PLANE + col * PITCH + row] = (unsigned short)mid;
            if (NP > 2) planes[2 * PLANE + col * PITCH + row] = (unsigned short)lo;
        }
        if (COT) {
            const float* g_b = g + (size_t)b * D;
            float* cot_b = cot + (size_t)b * (K + 1) * D;
            for (int row = tid; row < D; row += NT) {
                float acc = 0.0f;
                for (int k = 0; k < D; ++k) acc = fmaf(to_f32(a_last[row * D + k]), g_b[k], acc);
                vbuf[row] = acc;
                if (c0 == 0) {
                    cot_b[(size_t)K * D + row] = g_b[row];
                    cot_b[(size_t)(K - 1) * D + row] = acc;
                }
            }
        }
    }
    __syncthreads();
    if (K < 2) return;

    // lane's 64 bytes of chunk kc of mats[r]: row row0 + m, elements kc*K_PER_CHUNK + h*K_PER_LANE + [0, K_PER_LANE)
    auto load_raw = [&](u32x4 (&dst)[4], const Tin* base) {
#pragma unroll
        for (int q = 0; q < 4; ++q) dst[q] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(base) + 16 * q);
    };
    const Tin* a_lane = mats_b + (size_t)(row0 + m) * D + h * C::K_PER_LANE;  // + r*D*D + kc*K_PER_CHUNK
    u32x4 ring[RING][4];
#pragma unroll
    for (int c = 0; c < AHEAD; ++c) load_raw(ring[c], a_lane + (size_t)(K - 2) * D * D + c * C::K_PER_CHUNK);

    // byte offset of this lane's B fragments inside a plane: column m (+32 j), k = h*K_PER_LANE (+ chunk, + 8 t)
    const unsigned b_lane = (unsigned)(m * PITCH + h * C::K_PER_LANE) * 2;
    int cur = 0;  // vbuf parity
    for (int r = K - 2; r >= 0; --r) {
        f32x16 acc[2][2];  // [0]: hi*hi products, [1]: all smaller ones
#pragma unroll
        for (int o = 0; o < 2; ++o)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[o][j][e] = 0.0f;
        float vdot = 0.0f;
        u32x4 bfr[2][NP][2];
        auto load_b = [&](u32x4 (&dst)[NP][2], int k_off) {
#pragma unroll
            for (int sp = 0; sp < NP; ++sp) {
                const char* bp = smem + (size_t)sp * PLANE * 2 + b_lane + k_off * 2;
                dst[sp][0] = *reinterpret_cast<const u32x4*>(bp);
                dst[sp][1] = *reinterpret_cast<const u32x4*>(bp + 32 * PITCH * 2);
            }
        };
        load_b(bfr[0], 0);
        const Tin* a_r = a_lane + (size_t)r * D * D;
        const Tin* a_wrap = a_lane + (size_t)(r > 0 ? r - 1 : 0) * D * D;
        const float* v_old = vbuf + cur * D + h * C::K_PER_LANE;
#pragma unroll
        for (int kc = 0; kc < NCH; ++kc) {
            const int slot = kc % RING;
            const int ahead = kc + AHEAD;
            load_raw(ring[(slot + AHEAD) % RING],
                     ahead < NCH ? a_r + ahead * C::K_PER_CHUNK : a_wrap + (ahead - NCH) * C::K_PER_CHUNK);
            // A fragments of this chunk, one per plane and product step
            u32x4 afr[NA][C::T_STEPS];
            if (NA == 1) {
#pragma unroll
                for (int t = 0; t < C::T_STEPS; ++t) afr[0][t] = ring[slot][t];
            } else {
#pragma unroll
                for (int t = 0; t < C::T_STEPS; ++t)
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        const u32x4 raw = ring[slot][2 * t + (w >> 1)];
                        const float x0 = __uint_as_float(raw[2 * (w & 1)]), x1 = __uint_as_float(raw[2 * (w & 1) + 1]);
                        unsigned hi, mid, lo;
                        split2(x0, x1, hi, mid, lo);
                        afr[0][t][w] = hi;
                        afr[NA > 1 ? 1 : 0][t][w] = mid;
                        afr[NA > 2 ? 2 : 0][t][w] = lo;
                    }
            }
            if (COT) {
                const float* vk = v_old + kc * C::K_PER_CHUNK;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    if (NA == 1) {  // 8 bf16 per 16 bytes
                        const f32x4 va = *reinterpret_cast<const f32x4*>(vk + 8 * q);
                        const f32x4 vb = *reinterpret_cast<const f32x4*>(vk + 8 * q + 4);
                        const u32x4 raw = ring[slot][q];
                        vdot = fmaf(bf16_lo(raw[0]), va[0], vdot);
                        vdot = fmaf(bf16_hi(raw[0]), va[1], vdot);
                        vdot = fmaf(bf16_lo(raw[1]), va[2], vdot);
                        vdot = fmaf(bf16_hi(raw[1]), va[3], vdot);
                        vdot = fmaf(bf16_lo(raw[2]), vb[0], vdot);
                        vdot = fmaf(bf16_hi(raw[2]), vb[1], vdot);
                        vdot = fmaf(bf16_lo(raw[3]), vb[2], vdot);
                        vdot = fmaf(bf16_hi(raw[3]), vb[3], vdot);
                    } else {  // 4 floats per 16 bytes
                        const f32x4 va = *reinterpret_cast<const f32x4*>(vk + 4 * q);
                        const u32x4 raw = ring[slot][q];
#pragma unroll
                        for (int e = 0; e < 4; ++e) vdot = fmaf(__uint_as_float(raw[e]), va[e], vdot);
                    }
                }
            }
            // B fragments (3 planes x 2 column tiles) are read one product step ahead of use.
#pragma unroll
            for (int t = 0; t < C::T_STEPS; ++t) {
                const int u = kc * C::T_STEPS + t;           // product step within the suffix step
                const int slot_b = u & 1;
                if (u + 1 < NCH * C::T_STEPS) {
                    const int kc_n = (u + 1) / C::T_STEPS, t_n = (u + 1) % C::T_STEPS;
                    load_b(bfr[slot_b ^ 1], kc_n * C::K_PER_CHUNK + 8 * t_n);
                }
#pragma unroll
                for (int sp = NP - 1; sp >= 0; --sp)  // small planes first
#pragma unroll
                    for (int ap = NA - 1; ap >= 0; --ap) {
                        if (ap + sp > LBI_SPLIT_MAX_ORDER) continue;
                        const int o = ap + sp == 0 ? 0 : 1;
                        acc[o][0] = mma(afr[ap][t], bfr[slot_b][sp][0], acc[o][0]);
                        acc[o][1] = mma(afr[ap][t], bfr[slot_b][sp][1], acc[o][1]);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);
        }

        // Everyone is done reading S; form the new block, write it out and re-split it.
        lds_barrier();
        float* o_r = out_b + (size_t)r * D * D;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int gq = 0; gq < 4; ++gq) {
                float tot[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    tot[e] = acc[1][j][4 * gq + e] + acc[0][j][4 * gq + e];
                const int row = row0 + gq * 8 + h * 4;
                const int col = j * 32 + m;
                unsigned hi0, mid0, lo0, hi1, mid1, lo1;
                split2(tot[0], tot[1], hi0, mid0, lo0);
                split2(tot[2], tot[3], hi1, mid1, lo1);
                unsigned short* dst = planes + col * PITCH + row;
                *reinterpret_cast<u32x2*>(dst) = u32x2{hi0, hi1};
                *reinterpret_cast<u32x2*>(dst + PLANE) = u32x2{mid0, mid1};
                if (NP > 2) *reinterpret_cast<u32x2*>(dst + 2 * PLANE) = u32x2{lo0, lo1};
#pragma unroll
                for (int e = 0; e < 4; ++e) o_r[(size_t)(row + e) * D + c0 + col] = tot[e];
            }
        if (COT) {
            const float total = vdot + __shfl_xor(vdot, 32, 64);
            if (h == 0) {
                vbuf[(cur ^ 1) * D + row0 + m] = total;
                if (c0 == 0) cot[((size_t)b * (K + 1) + r) * D + row0 + m] = total;
            }
        }
        lds_barrier();
        cur ^= 1;
    }
}

template <typename Tin, int NP>
int launch_planes(const void* mats, void* out, const void* g, void* cot, int B, int K, hipStream_t stream) {
    const size_t lds_bytes = (size_t)NP * PLANE * 2 + (cot ? 2 * D * sizeof(float) : 0);
    const dim3 grid(((B + 7) / 8) * 8 * NB);
    if (cot) {
        auto kern = scan_split_kernel<Tin, true, NP>;
        if (int rc = ensure_dynamic_lds<&scan_split_kernel<Tin, true, NP>>(lds_bytes)) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(NT), lds_bytes, stream, static_cast<const Tin*>(mats),
                           static_cast<float*>(out), static_cast<const float*>(g), static_cast<float*>(cot), B, K);
    } else {
        auto kern = scan_split_kernel<Tin, false, NP>;
        if (int rc = ensure_dynamic_lds<&scan_split_kernel<Tin, false, NP>>(lds_bytes)) return rc;
        hipLaunchKernelGGL(kern, grid, dim3(NT), lds_bytes, stream, static_cast<const Tin*>(mats),
                           static_cast<float*>(out), static_cast<const float*>(nullptr), static_cast<float*>(nullptr),
                           B, K);
    }
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

// planes: 3 = exact; 2 = 16-bit suffix operand, bf16 storage only (fp32 storage always runs exact).
template <typename Tin>
int launch(const void* mats, void* out, const void* g, void* cot, int B, int K, int planes, hipStream_t stream) {
    if (planes < 3 && Chunk<Tin>::NA == 1) return launch_planes<Tin, 2>(mats, out, g, cot, B, K, stream);
    return launch_planes<Tin, 3>(mats, out, g, cot, B, K, stream);
}

}  // namespace scan_split
}  // namespace lbi
