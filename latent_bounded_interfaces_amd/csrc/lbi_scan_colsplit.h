// Suffix scan for d = 256 with bf16 storage: column-owner form of the exact three-way split.
//
// S_r = A_r S_{r+1}.  Here a WAVE owns 16 columns of the running suffix S for all 256 rows, so the
// operand that changes every step (S) never leaves the wave: the wave re-splits its own 256 x 16 result
// into three bf16 planes (hi + mid + lo == the fp32 value exactly, see lbi_scan_split.h) and turns it from
// the accumulator layout (lane = column, 4 rows per lane group) into the B-operand layout (8 consecutive
// rows per lane group) with two lane-group swaps per register (v_permlane32_swap, v_permlane16_swap): no
// LDS, no workgroup barrier between steps, and the B fragments of a whole step (8 k-steps x 3 planes) stay
// in registers.  The operand every wave needs, the bf16 matrix A_r, is streamed once per workgroup through
// LDS by global_load_lds in chunks of 64 k-columns (256 rows x 128 bytes; four-slot ring, three chunks
// ahead, one barrier per chunk), XOR-swizzled on 16-byte pieces so the 16x16x32 A-fragment reads are
// conflict free.  A workgroup is four waves = 64 columns of one batch element (one workgroup per CU, one
// wave per SIMD); the four column blocks of a batch element sit on one XCD and share A in its L2.
//
// The loop runs k-chunk major, row tiles inner, so a row tile is complete after the products of the last
// chunk and its store / split / swap work is written right behind them: it runs under the products of the
// following tiles, and the first k-steps of the next step find their fragments ready.
//
// Per wave and step: 16 row tiles x 8 k-steps x 3 planes = 384 v_mfma_f32_16x16x32_bf16, 128 A-fragment
// reads (one per three products), one fp32 accumulator per tile (the summation order of an fp32 dot
// product with the three planes of a k-step taken small first).
//
// COT: the cotangent chain v_r = A_r v_{r+1} rides along on four more waves per workgroup (one per SIMD).  The four
// workgroups of a batch element each own 64 entries of every v_r (workgroup = column block c <-> entries 64 c ..
// 64 c + 63): four lanes of a chain wave share one row of A_r, read it from the chunks the matrix waves stream
// through LDS anyway (no extra memory traffic) and sum 16 partial dot products of 16 terms in fp32.  The vector is exchanged between
// the four workgroups through the result array cot[b, r, :] itself: it is filled with a marker word before the
// launch, the owner stores its 64 entries, the others poll until the word differs from the marker (agent-scope
// atomics; see cotangent256_group_kernel in lbi_scan.hip for the protocol and its bounded wait).  The entries of
// v_{r+1} arrive some microseconds into step r, so the chain waves keep the chunks of their rows in registers and
// multiply in the last quarter of the step, after one of them has picked the vector up.  The chain waves take part
// in the chunk barriers and never wait for memory they do not expect to be there already.
#pragma once

#include "lbi_common.h"

namespace lbi {
namespace scan_col {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

constexpr int D = 256, NWAVE = 4, NT = 64 * NWAVE, CB = 16 * NWAVE, NB = D / CB;
constexpr int MT = D / 16, KS = D / 32;
constexpr int CHUNK_K = 64, NCHUNK = D / CHUNK_K, CHUNK_KS = CHUNK_K / 32;  // k-steps per chunk
constexpr int ROW_BYTES = D * 2, CHUNK_ROW_BYTES = CHUNK_K * 2, CHUNK_BYTES = D * CHUNK_ROW_BYTES;  // 32 KB
constexpr int NDMA = CHUNK_BYTES / 1024 / NWAVE;  // 1 KB transfers per wave and chunk
constexpr int LDS_BYTES = NCHUNK * CHUNK_BYTES;   // 128 KB

constexpr int waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

__device__ __forceinline__ void dma16_at(const void* lane_ptr, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(lane_ptr)
                 : "memory");
}

__device__ __forceinline__ unsigned pack_bf16(float lo, float hi) {
    const f32x2 v = {lo, hi};
    return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ float bf16_lo(unsigned w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16_hi(unsigned w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ void split2(float x0, float x1, unsigned& hi, unsigned& mid, unsigned& lo) {
    hi = pack_bf16(x0, x1);
    const float r0 = x0 - bf16_lo(hi), r1 = x1 - bf16_hi(hi);
    mid = pack_bf16(r0, r1);
    lo = pack_bf16(r0 - bf16_lo(mid), r1 - bf16_hi(mid));
}

// hi and mid only: x rounded to 16 significand bits
__device__ __forceinline__ void split2_top(float x0, float x1, unsigned& hi, unsigned& mid) {
    hi = pack_bf16(x0, x1);
    mid = pack_bf16(x0 - bf16_lo(hi), x1 - bf16_hi(hi));
}

__device__ __forceinline__ f32x4 mma(u32x4 a, u32x4 b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0,
                                                   0);
}

// NP = planes of the running suffix that enter the products: 3 is exact (the fp32 value), 2 rounds the operand to
// 16 significand bits (hi + mid); the accumulation and the stored result are fp32 either way.
constexpr unsigned kChainMarker = 0x7fa5c3e1u;  // a NaN payload no arithmetic produces: "not written yet"

// The chain waves of scan_colsplit_kernel<NP, true> (see the file comment): four per workgroup, one per SIMD, so that
// their vector work spreads evenly under the matrix waves.  `part` = this workgroup's column block = its 64 entries
// of the chain vector; chain wave cw owns rows 16 cw .. 16 cw + 15 of them, four lanes per row, a quarter of every
// chunk's 64 k each (two 16-byte pieces).  They execute exactly the barriers of the matrix waves: four per step.
__device__ __forceinline__ void chain_wave(const char* smem, float* vbuf, const bf16_raw* __restrict__ mats_b,
                                           const float* __restrict__ g_b, float* __restrict__ cot_b, int part,
                                           int cw, int lane, int K, int spin_limit) {
    const int row = 64 * part + 16 * cw + (lane >> 2);   // this lane's row of every matrix, its entry of every vector
    const int q = lane & 3;                              // its quarter of a chunk's k range
    auto vb = [&](int r) { return vbuf + (r % 3) * D; };
    auto chunk_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    // one entry of A_r v_{r+1} straight from memory: the first vector, and the way out of a wait that ran out
    auto entry_from_memory = [&](int r, int idx, const float* v) {
        const bf16_raw* a_row = mats_b + (size_t)r * D * D + (size_t)idx * D;
        float acc = 0.0f;
        for (int k = 0; k < D; k += 4) {
            const f32x4 a4 = load4(a_row + k);
            const f32x4 v4 = *reinterpret_cast<const f32x4*>(v + k);
            acc = fmaf(a4[3], v4[3], fmaf(a4[2], v4[2], fmaf(a4[1], v4[1], fmaf(a4[0], v4[0], acc))));
        }
        return acc;
    };
    auto publish = [&](int r, float value) {
        unsigned bits = __float_as_uint(value);
        if (bits == kChainMarker) bits = 0x7fc00000u;
        vb(r)[row] = __uint_as_float(bits);
        __hip_atomic_store(reinterpret_cast<unsigned*>(cot_b + (size_t)r * D + row), bits, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    };
    // the 192 entries of v_r the partners own, three per lane of chain wave 0: polled until written (or formed here
    // after `spin_limit` polls), then into the LDS copy
    auto collect = [&](int r) {
        unsigned* words = reinterpret_cast<unsigned*>(cot_b + (size_t)r * D);
        int idx[3];
        unsigned got[3] = {kChainMarker, kChainMarker, kChainMarker};
#pragma unroll
        for (int e = 0; e < 3; ++e) {
            const int f = lane + 64 * e;
            idx[e] = f < 64 * part ? f : f + 64;
        }
        int spins = 0;
        while (true) {
            bool all = true;
#pragma unroll
            for (int e = 0; e < 3; ++e)
                if (got[e] == kChainMarker) {
                    got[e] = __hip_atomic_load(words + idx[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    all = all && got[e] != kChainMarker;
                }
            if (all) break;
            if (++spins > spin_limit) {
#pragma unroll
                for (int e = 0; e < 3; ++e)
                    if (got[e] == kChainMarker) got[e] = __float_as_uint(entry_from_memory(r, idx[e], vb(r + 1)));
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
#pragma unroll
        for (int e = 0; e < 3; ++e) vb(r)[idx[e]] = __uint_as_float(got[e]);
    };
    // the lane's two pieces (16 k) of chunk slot c; the pieces of a row are XOR-swizzled as the DMA laid them down
    auto read_pieces = [&](u32x4 (&dst)[2], int c) {
        const char* base = smem + c * CHUNK_BYTES + row * CHUNK_ROW_BYTES;
#pragma unroll
        for (int t = 0; t < 2; ++t)
            dst[t] = *reinterpret_cast<const u32x4*>(base + (((2 * q + t) ^ ((row >> 1) & 7)) << 4));
    };
    // 16 terms; v points at the lane's k range of the chunk
    auto dot = [&](const u32x4 (&a)[2], const float* v) {
        float acc = 0.0f;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const f32x4 lo = *reinterpret_cast<const f32x4*>(v + 8 * t);
            const f32x4 hi = *reinterpret_cast<const f32x4*>(v + 8 * t + 4);
            acc = fmaf(bf16_lo(a[t][0]), lo[0], acc);
            acc = fmaf(bf16_hi(a[t][0]), lo[1], acc);
            acc = fmaf(bf16_lo(a[t][1]), lo[2], acc);
            acc = fmaf(bf16_hi(a[t][1]), lo[3], acc);
            acc = fmaf(bf16_lo(a[t][2]), hi[0], acc);
            acc = fmaf(bf16_hi(a[t][2]), hi[1], acc);
            acc = fmaf(bf16_lo(a[t][3]), hi[2], acc);
            acc = fmaf(bf16_hi(a[t][3]), hi[3], acc);
        }
        return acc;
    };

    // v_K = g (chain wave 0 keeps a copy and writes the owner's 64 entries of the result); v_{K-1} = A_{K-1} g, one
    // lane per row, from memory
    if (cw == 0) {
        *reinterpret_cast<f32x4*>(vb(K) + 4 * lane) = *reinterpret_cast<const f32x4*>(g_b + 4 * lane);
        cot_b[(size_t)K * D + 64 * part + lane] = g_b[64 * part + lane];
    }
    if (q == 0) publish(K - 1, entry_from_memory(K - 1, row, g_b));
    for (int r = K - 2; r >= 0; --r) {
        // The chunks of A_r pass through LDS one window each; v_{r+1} is complete in LDS only at the last barrier of
        // the step (chain wave 0 picks the partners' entries up in the third window), so the pieces of the first
        // three chunks wait in registers and all products are formed in the last window.
        u32x4 piece[4][2];
        chunk_barrier();
        read_pieces(piece[0], 0);
        chunk_barrier();
        read_pieces(piece[1], 1);
        chunk_barrier();
        read_pieces(piece[2], 2);
        if (cw == 0) collect(r + 1);                     // written by the partners at the end of the step before
        chunk_barrier();
        read_pieces(piece[3], 3);
        const float* v = vb(r + 1) + 16 * q;
        float acc = (dot(piece[0], v) + dot(piece[1], v + 64)) + (dot(piece[2], v + 128) + dot(piece[3], v + 192));
        acc += __shfl_xor(acc, 1, 64);
        acc += __shfl_xor(acc, 2, 64);
        if (q == 0) publish(r, acc);
    }
}

template <int NP, bool COT>
__global__ __launch_bounds__(COT ? 2 * NT : NT) void scan_colsplit_kernel(
    const bf16_raw* __restrict__ mats, float* __restrict__ out, const float* __restrict__ g_in,
    float* __restrict__ cot, int B, int K, int spin_limit) {
    extern __shared__ __align__(16) char smem[];
    const int id = blockIdx.x;
    const int slot_id = id >> 3;
    const int b = (slot_id / NB) * 8 + (id & 7);
    if (b >= B) return;
    const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    if (COT && wave >= NWAVE) {
        chain_wave(smem, reinterpret_cast<float*>(smem + LDS_BYTES), mats + (size_t)b * K * D * D,
                   g_in + (size_t)b * D, cot + (size_t)b * (K + 1) * D, slot_id % NB, wave - NWAVE, lane, K,
                   spin_limit);
        return;
    }
    const int col = (slot_id % NB) * CB + wave * 16 + n;  // this lane's column of S
    const bf16_raw* mats_b = mats + (size_t)b * K * D * D;
    float* out_b = out + (size_t)b * (K + 1) * D * D;
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem;

    // A chunk in LDS: 256 rows of 128 bytes; piece p (16 bytes) of row i sits at piece p ^ ((i >> 1) & 7), so the
    // 16 rows a fragment read touches (128-byte stride) cover all 64 banks once.
    // Fragment of this lane, k-step s of the chunk, row tile mt: row 16 mt + n, piece 4 s + g.
    unsigned frag_off[CHUNK_KS];
#pragma unroll
    for (int s = 0; s < CHUNK_KS; ++s) frag_off[s] = (unsigned)(n * CHUNK_ROW_BYTES + (((4 * s + g) ^ (n >> 1)) << 4));
    // Transfers of this wave: x-th kilobyte of its share = rows 8 (NDMA wave + x) + (lane >> 3), landing piece lane & 7.
    unsigned dma_src[NDMA];
#pragma unroll
    for (int x = 0; x < NDMA; ++x) {
        const int row = 8 * (NDMA * wave + x) + (lane >> 3);
        dma_src[x] = (unsigned)(row * ROW_BYTES + (((lane & 7) ^ ((row >> 1) & 7)) << 4));
    }
    auto issue_chunk = [&](int r, int c) __attribute__((always_inline)) {
        const char* src = reinterpret_cast<const char*>(mats_b + (size_t)r * D * D) + c * CHUNK_ROW_BYTES;
#pragma unroll
        for (int x = 0; x < NDMA; ++x)
            dma16_at(src + dma_src[x], lds0 + c * CHUNK_BYTES + 1024 * (NDMA * wave + x));
    };

    f32x4 acc[MT];
    u32x4 bfr[KS][NP];      // B fragments of the current step: [k-step][plane]
    u32x4 late[2][NP];      // fragments of the last two k-steps of the next step, until this step is done with its own
    u32x2 even_words[NP];   // packed planes of the even tile of a pair, waiting for the odd one

    // Row tile mt of step r is complete in acc: store it, split it, and with its pair partner form the B fragments of
    // k-step mt / 2 of the next step.  Accumulator layout: lane (n, g), register e <-> row 16 mt + 4 g + e; fragment
    // layout: lane (n, g) <-> rows 32 ks + 8 g .. + 7.  With P / Q the registers of tiles 2 ks / 2 ks + 1,
    // permlane32_swap then permlane16_swap leaves rows (g: P0 P2 Q0 Q2) in one register and (P1 P3 Q1 Q3) in the other.
    auto finish_tile = [&](int mt, int r, bool hold_late) __attribute__((always_inline)) {
        float* o_r = out_b + (size_t)r * D * D + (size_t)(16 * mt + 4 * g) * D + col;
        const f32x4 tot = acc[mt];
#pragma unroll
        for (int e = 0; e < 4; ++e) o_r[(size_t)e * D] = tot[e];
        unsigned w[3][2];
        if (NP == 3) {
            split2(tot[0], tot[1], w[0][0], w[1][0], w[2][0]);
            split2(tot[2], tot[3], w[0][1], w[1][1], w[2][1]);
        } else {
            split2_top(tot[0], tot[1], w[0][0], w[1][0]);
            split2_top(tot[2], tot[3], w[0][1], w[1][1]);
        }
        if ((mt & 1) == 0) {
#pragma unroll
            for (int p = 0; p < NP; ++p) even_words[p] = u32x2{w[p][0], w[p][1]};
            return;
        }
        const int ks = mt >> 1;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            u32x4 frag;
#pragma unroll
            for (int hw = 0; hw < 2; ++hw) {
                const u32x2 a = __builtin_amdgcn_permlane32_swap(even_words[p][hw], w[p][hw], false, false);
                const u32x2 c = __builtin_amdgcn_permlane16_swap(a[0], a[1], false, false);
                frag[hw] = c[0];
                frag[2 + hw] = c[1];
            }
            if (hold_late && ks >= KS - CHUNK_KS) late[ks - (KS - CHUNK_KS)][p] = frag;
            else bfr[ks][p] = frag;
        }
    };

    // First suffix S_{K-1} = A_{K-1}, and the identity tail.
    {
        const bf16_raw* a_last = mats_b + (size_t)(K - 1) * D * D;
        float* o_eye = out_b + (size_t)K * D * D;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int row = 16 * mt + 4 * g + e;
                acc[mt][e] = to_f32(a_last[(size_t)row * D + col]);
                o_eye[(size_t)row * D + col] = row == col ? 1.0f : 0.0f;
            }
    }
    if (K >= 2) {
#pragma unroll
        for (int c = 0; c < NCHUNK - 1; ++c) issue_chunk(K - 2, c);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) finish_tile(mt, K - 1, false);

    const f32x4 zero = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int r = K - 2; r >= 0; --r) {
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            // Chunk c of this step was issued three chunks ago.  Younger than it: the two chunks issued since
            // (2 NDMA transfers) and, except before the last chunk, the 64 stores of the step before, which alone
            // exceed the 63 operations that can be outstanding, so only the last chunk needs an explicit count.
            if (r == K - 2 && c == 0) {
                __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));  // the three chunks issued before the loop
            } else if (c == NCHUNK - 1) {
                if (r > 0) __builtin_amdgcn_s_waitcnt(waitcnt_vm(2 * NDMA));
                else __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
            }
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            // slot of chunk c - 1 is free now: refill it with the chunk three ahead
            if (c == 0) {
                issue_chunk(r, NCHUNK - 1);
            } else if (r > 0) {
                issue_chunk(r - 1, c - 1);
            }
            const char* stage = smem + c * CHUNK_BYTES;
            // k-step outer, four row tiles at a time: the three planes of a tile (small first) go into one
            // accumulator, and consecutive products never share it
#pragma unroll
            for (int s = 0; s < CHUNK_KS; ++s) {
                const int ks = c * CHUNK_KS + s;
                const bool first = c == 0 && s == 0;
#pragma unroll
                for (int mt = 0; mt < MT; mt += 4) {
                    u32x4 a[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        a[t] = *reinterpret_cast<const u32x4*>(stage + (mt + t) * 16 * CHUNK_ROW_BYTES + frag_off[s]);
#pragma unroll
                    for (int p = NP - 1; p >= 0; --p)
#pragma unroll
                        for (int t = 0; t < 4; ++t)
                            acc[mt + t] = mma(a[t], bfr[ks][p], (first && p == NP - 1) ? zero : acc[mt + t]);
                    if (c == NCHUNK - 1 && s == CHUNK_KS - 1) {
#pragma unroll
                        for (int t = 0; t < 4; ++t) finish_tile(mt + t, r, true);
                    }
                }
            }
        }
#pragma unroll
        for (int s = 0; s < CHUNK_KS; ++s)
#pragma unroll
            for (int p = 0; p < NP; ++p) bfr[KS - CHUNK_KS + s][p] = late[s][p];
    }
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
}

template <int NP, bool COT>
int launch_planes(const void* mats, void* out, const void* g, void* cot, int B, int K, int spin_limit,
                  hipStream_t stream) {
    constexpr size_t lds_bytes = LDS_BYTES + (COT ? 3 * D * sizeof(float) : 0);   // + three copies of the chain vector
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");
    auto kern = scan_colsplit_kernel<NP, COT>;
    if (int rc = ensure_dynamic_lds<&scan_colsplit_kernel<NP, COT>>(lds_bytes)) return rc;
    const dim3 grid(((B + 7) / 8) * 8 * NB);
    hipLaunchKernelGGL(kern, grid, dim3(COT ? 2 * NT : NT), lds_bytes, stream, static_cast<const bf16_raw*>(mats),
                       static_cast<float*>(out), static_cast<const float*>(g), static_cast<float*>(cot), B, K,
                       spin_limit);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

// Matrices only.
inline int launch(const void* mats, void* out, int B, int K, int planes, hipStream_t stream) {
    return planes >= 3 ? launch_planes<3, false>(mats, out, nullptr, nullptr, B, K, 0, stream)
                       : launch_planes<2, false>(mats, out, nullptr, nullptr, B, K, 0, stream);
}

// Matrices and the cotangent chain; `cot` must have been filled with kChainMarker on `stream` before.  Only for
// batches whose 4 B workgroups are all resident at once (the chain waves of a batch element wait for each other).
inline int launch_with_chain(const void* mats, void* out, const void* g, void* cot, int B, int K, int planes,
                             int spin_limit, hipStream_t stream) {
    return planes >= 3 ? launch_planes<3, true>(mats, out, g, cot, B, K, spin_limit, stream)
                       : launch_planes<2, true>(mats, out, g, cot, B, K, spin_limit, stream);
}

}  // namespace scan_col
}  // namespace lbi
