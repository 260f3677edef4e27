// dQ kernel of the attention input-pullback (fp16 / bf16 storage, head dim 64 or 128).
//
// One wave owns 32 queries and PB directions (at head dim 128 the 256 accumulation registers
// are exactly its four dQ tiles of 32 x 128; head dim 64 has room for eight); a workgroup is
// 4 waves = 128 queries.
//   S^T  = K Q^T        A = K tile (LDS, shared), B = Q (registers)   lanes = queries, registers = keys
//   P    = exp2(S^T c - lse2), once for the four directions
//   dP^T = V dO_p^T     A = V tile (LDS, shared), B = dO_p (LDS, private to the wave)
//   dS_p = P (dP_p - delta_p)       delta_p = rowsum(dO_p o O), formed by this kernel and left for the dK/dV kernel
//   dQ_p += dS_p K      A = dS_p (registers), B = K tile through transpose reads
// K/V tiles of 32 keys arrive by global_load_lds into a two-stage ring (loop unrolled by
// two, stage offsets are immediates); the wave's four d_out tiles are copied to LDS once.
// S^T and dP^T tiles use VGPR-form MFMAs; the dS work of direction p is written between
// the dP products of direction p+1 so it runs while the matrix pipe is busy.  Causal
// masking is confined to the last four steps of a workgroup.
#pragma once

#include "lbi_attn_dkdv128.h"

#ifndef LBI_DQ_GRING
#define LBI_DQ_GRING 2
#endif

namespace lbi {
namespace attn_mfma {

template <typename T, int DH, int PB, bool CAUSAL>
__global__ __launch_bounds__(256) void dq_ring_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                    const T* __restrict__ v, const T* __restrict__ d_out,
                                                    const float* __restrict__ lse2, const float* __restrict__ o32,
                                                    float* __restrict__ delta, T* __restrict__ dq, int n_bh, int H,
                                                    int P, int T_len, float scale) {
    constexpr int KS = DH / 16, ND = DH / 32;
    constexpr int RB = DH * 2;               // bytes per tile row
    constexpr int CPR = DH / 8;              // 16-byte chunks per tile row
    constexpr int NX = DH / 64;              // global_load_lds per tile per wave
    static_assert(KS >= 4 && PB * ND <= 16, "four VALU blocks per direction; 256 accumulation registers");
    constexpr unsigned TILE = 32 * RB;       // 8 KiB (Dh 128) / 4 KiB (Dh 64)
    constexpr unsigned STAGE = 2 * TILE;     // K tile, V tile
    constexpr unsigned GF0 = 2 * STAGE;      // then [4 waves][PB] d_out tiles
    extern __shared__ __align__(16) char smem[];

    const int n_qb = (T_len + 127) / 128;
    const int n_pb = (P + PB - 1) / PB;
    int bh, rem;
    if (!map_block(n_qb * n_pb, n_bh, bh, rem)) return;
    const int qb = n_qb - 1 - rem / n_pb;  // longest rows first
    const int p0 = (rem % n_pb) * PB;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, m = lane & 31, h = lane >> 5;
    const bool active = qb * 128 + wave * 32 < T_len;
    const int i0w = min(qb * 128 + wave * 32, T_len - 32);
    const size_t base = (size_t)bh * T_len * DH;
    const T* k_bh = k + base;
    const T* v_bh = v + base;

    const unsigned lane_nat = m * RB + ((h ^ swz<DH>(m)) << 4);  // ^ (ks << 5)
    const unsigned s16 = lane & 15, g1 = (lane >> 4) & 1;
    const unsigned tr_row = 4 * h + (s16 >> 2), tr_chunk = 2 * g1 + ((s16 & 3) >> 1);
    const unsigned lane_tr = tr_row * RB + ((tr_chunk ^ swz<DH>(tr_row)) << 4) + ((s16 & 1) << 3);

    unsigned dma_off[NX];
#pragma unroll
    for (int x = 0; x < NX; ++x) {
        const int sigma = 64 * (NX * wave + x) + lane;
        const int r = sigma / CPR;
        dma_off[x] = r * RB + (((sigma % CPR) ^ swz<DH>(r)) << 4);
    }
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem;
    auto issue_tile = [&](int j_row, unsigned stage_base) __attribute__((always_inline)) {
        const unsigned row_bytes = (unsigned)j_row * RB;
#pragma unroll
        for (int x = 0; x < NX; ++x) {
            dma16(k_bh, row_bytes + dma_off[x], lds0 + stage_base + 1024 * (NX * wave + x));
            dma16(v_bh, row_bytes + dma_off[x], lds0 + stage_base + TILE + 1024 * (NX * wave + x));
        }
    };

    // Resident: Q fragments (B operand of S^T), lse2 and delta of the lane's query.  delta_p[i] = sum_d
    // d_out_p[i][d] O[i][d] is formed here, from the d_out tiles the wave has just put into LDS and the forward
    // output row of the lane's query (two lanes per query, half the head dim each), and left in the workspace
    // (negated) for the dK/dV kernel: every (direction, query) has exactly one owner wave.
    u32x4 qf[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
        qf[ks] = *reinterpret_cast<const u32x4*>(q + base + (size_t)(i0w + m) * DH + 16 * ks + 8 * h);
    const float my_lse = lse2[(size_t)bh * T_len + i0w + m];
    float my_delta[PB];
    char* gf_w = smem + GF0 + wave * PB * TILE;
#pragma unroll
    for (int pp = 0; pp < PB; ++pp) {
        const int p = min(p0 + pp, P - 1);  // surplus slots redo the last direction; never stored
        const size_t row0 = (((size_t)b * P + p) * H + hh) * T_len + i0w;
#pragma unroll
        for (int u = 0; u < CPR / 2; ++u) {
            const int slot = 64 * u + lane;
            const int r = slot / CPR, c = slot % CPR;
            const u32x4 val = *reinterpret_cast<const u32x4*>(d_out + (row0 + r) * DH + 8 * c);
            *reinterpret_cast<u32x4*>(gf_w + pp * TILE + tile_off<DH>(r, c)) = val;
        }
        my_delta[pp] = 0.0f;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");  // the tiles are the wave's own: LDS runs in order
    __builtin_amdgcn_wave_barrier();
    {
        const float* o_row = o32 + base + (size_t)(i0w + m) * DH + h * (DH / 2);
#pragma unroll
        for (int c = 0; c < CPR / 2; ++c) {
            const f32x4 o_lo = *reinterpret_cast<const f32x4*>(o_row + 8 * c);
            const f32x4 o_hi = *reinterpret_cast<const f32x4*>(o_row + 8 * c + 4);
#pragma unroll
            for (int pp = 0; pp < PB; ++pp) {
                const u32x4 g4 = *reinterpret_cast<const u32x4*>(gf_w + pp * TILE + tile_off<DH>(m, h * (CPR / 2) + c));
                float part = my_delta[pp];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    part = fmaf(Mma<T>::lo(g4[e]), o_lo[2 * e], part);
                    part = fmaf(Mma<T>::hi(g4[e]), o_lo[2 * e + 1], part);
                }
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    part = fmaf(Mma<T>::lo(g4[2 + e]), o_hi[2 * e], part);
                    part = fmaf(Mma<T>::hi(g4[2 + e]), o_hi[2 * e + 1], part);
                }
                my_delta[pp] = part;
            }
        }
#pragma unroll
        for (int pp = 0; pp < PB; ++pp) {
            my_delta[pp] += __shfl_xor(my_delta[pp], 32, 64);
            if (active && h == 0 && p0 + pp < P)
                delta[(((size_t)b * P + p0 + pp) * H + hh) * T_len + i0w + m] = -my_delta[pp];  // kept negated
        }
    }

    f32x16 acc[PB][ND];
#pragma unroll
    for (int pp = 0; pp < PB; ++pp)
#pragma unroll
        for (int nd = 0; nd < ND; ++nd) acc[pp][nd] = zero16();
    const float sc2 = scale * LOG2E;

    auto tr_frag = [&](const char* tile, int kk, int nd) __attribute__((always_inline)) {
        typedef __attribute__((address_space(3))) s16x4* lds_ptr;
        const s16x4 lo =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + (lane_tr ^ (nd << 6)) + (16 * kk) * RB));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_ptr)(tile + (lane_tr ^ ((nd << 6) | 32)) + (16 * kk + 8) * RB));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        return u32x4{l2[0], l2[1], h2[0], h2[1]};
    };
    auto nat = [&](const char* tile, int ks) __attribute__((always_inline)) {
        return *reinterpret_cast<const u32x4*>(tile + (lane_nat ^ (ks << 5)));
    };

    // One key-tile step on the stage at byte offset SB.  thr: element 8g+e (key row) is
    // above the diagonal for this lane's query iff 8g + e > thr.
    auto step = [&](auto mask_tag, auto stage_tag, int thr) __attribute__((always_inline)) {
        constexpr bool MASK = decltype(mask_tag)::value;
        constexpr unsigned SB = decltype(stage_tag)::value;
        const char* kt = smem + SB;
        const char* vt = smem + SB + TILE;

        // ---- S^T, all eight K fragments in flight, then the V fragments (kept for 4 directions)
        u32x4 ka[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) ka[ks] = nat(kt, ks);
        f32x16 s = Mma<T>::mma_v_start(ka[0], qf[0]);
#pragma unroll
        for (int ks = 1; ks < KS; ++ks) Mma<T>::mma_v(ka[ks], qf[ks], s);
        u32x4 va[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) va[ks] = nat(vt, ks);
        // d_out fragment ring: fragment f = pp * KS + ks lives in slot f % GR and is fetched GR - 1 products ahead
        // (an LDS read issued one product ahead arrives after that product has drained)
        constexpr int GR = LBI_DQ_GRING;
        u32x4 gfr[GR];
        auto fetch_gf = [&](int f) __attribute__((always_inline)) {
            if (f < PB * KS) gfr[f % GR] = nat(gf_w + (f / KS) * TILE, f % KS);
        };
#pragma unroll
        for (int f = 0; f < GR - 1; ++f) fetch_gf(f);
        mma_v_settle(s);

        u32x4 pq[2];           // P rounded to the storage type
        u32x4 dsa[PB][2];      // dS_p, A operands of the dQ products
        f32x16 dp_prev = s;    // placeholder until the first dP tile exists
#pragma unroll
        for (int pp = 0; pp < PB; ++pp) {
            f32x16 dp;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int f = pp * KS + ks, cur = f % GR;
                fetch_gf(f + GR - 1);
                if (ks == 0) dp = Mma<T>::mma_v_start(va[0], gfr[cur]);
                else Mma<T>::mma_v(va[ks], gfr[cur], dp);
                // VALU work slotted under this product: P for pp == 0, dS_{pp-1} otherwise;
                // two (g) blocks of four elements per product for ks < 2 ... spread over ks 0..3
                if (ks < 4) {
                    const int g = ks;
                    if (pp == 0) {
                        float pr[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            pr[e] = __builtin_amdgcn_exp2f(s[4 * g + e] * sc2 - my_lse);
                            if (MASK && (8 * g + e > thr)) pr[e] = 0.0f;
                        }
                        unsigned w0 = Mma<T>::pack2(pr[0], pr[1]), w1 = Mma<T>::pack2(pr[2], pr[3]);
                        pin_here(w0, w1);
                        pq[g >> 1][2 * (g & 1)] = w0;
                        pq[g >> 1][2 * (g & 1) + 1] = w1;
                    } else {
                        const unsigned q0 = pq[g >> 1][2 * (g & 1)], q1 = pq[g >> 1][2 * (g & 1) + 1];
                        const float dl = my_delta[pp - 1];
                        const float d0 = Mma<T>::lo(q0) * (dp_prev[4 * g + 0] - dl);
                        const float d1 = Mma<T>::hi(q0) * (dp_prev[4 * g + 1] - dl);
                        const float d2 = Mma<T>::lo(q1) * (dp_prev[4 * g + 2] - dl);
                        const float d3 = Mma<T>::hi(q1) * (dp_prev[4 * g + 3] - dl);
                        unsigned w0 = Mma<T>::pack2(d0, d1), w1 = Mma<T>::pack2(d2, d3);
                        pin_here(w0, w1);
                        dsa[pp - 1][g >> 1][2 * (g & 1)] = w0;
                        dsa[pp - 1][g >> 1][2 * (g & 1) + 1] = w1;
                    }
                }
            }
            mma_v_settle(dp);
            dp_prev = dp;
        }
        // dS of the last direction, then the dQ products.
        u32x4 kfr[2];
        kfr[0] = tr_frag(kt, 0, 0);
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const unsigned q0 = pq[g >> 1][2 * (g & 1)], q1 = pq[g >> 1][2 * (g & 1) + 1];
            const float dl = my_delta[PB - 1];
            const float d0 = Mma<T>::lo(q0) * (dp_prev[4 * g + 0] - dl);
            const float d1 = Mma<T>::hi(q0) * (dp_prev[4 * g + 1] - dl);
            const float d2 = Mma<T>::lo(q1) * (dp_prev[4 * g + 2] - dl);
            const float d3 = Mma<T>::hi(q1) * (dp_prev[4 * g + 3] - dl);
            dsa[PB - 1][g >> 1][2 * (g & 1)] = Mma<T>::pack2(d0, d1);
            dsa[PB - 1][g >> 1][2 * (g & 1) + 1] = Mma<T>::pack2(d2, d3);
        }
#pragma unroll
        for (int i = 0; i < 2 * ND; ++i) {
            const int kk = i / ND, nd = i % ND, cur = i & 1;
            if (i + 1 < 2 * ND) kfr[cur ^ 1] = tr_frag(kt, (i + 1) / ND, (i + 1) % ND);
#pragma unroll
            for (int pp = 0; pp < PB; ++pp) acc[pp][nd] = Mma<T>::mma(dsa[pp][kk], kfr[cur], acc[pp][nd]);
        }
    };

    const int j_end = CAUSAL ? min(T_len, qb * 128 + 128) : T_len;
    const int n_it = j_end / 32;                       // even
    const int n_plain = CAUSAL ? max(0, n_it - 4) : n_it;  // steps wholly below the diagonal
    issue_tile(0, 0);
    auto two_steps = [&](auto mask_tag, int it) __attribute__((always_inline)) {
        const int j0 = it * 32;
        const int thr = i0w + m - j0 - 4 * h;
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
        __syncthreads();
        issue_tile(min(j0 + 32, T_len - 32), STAGE);
        step(mask_tag, std::integral_constant<unsigned, 0>{}, thr);
        __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));
        __syncthreads();
        issue_tile(min(j0 + 64, T_len - 32), 0);
        step(mask_tag, std::integral_constant<unsigned, STAGE>{}, thr - 32);
    };
    int it = 0;
    for (; it < n_plain; it += 2) two_steps(std::false_type{}, it);
    for (; it < n_it; it += 2) two_steps(std::true_type{}, it);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));

    if (active) {
#pragma unroll
        for (int pp = 0; pp < PB; ++pp) {
            if (p0 + pp >= P) break;
            unsigned short* o =
                reinterpret_cast<unsigned short*>(dq + ((((size_t)b * P + p0 + pp) * H + hh) * T_len + i0w) * DH);
#pragma unroll
            for (int nd = 0; nd < ND; ++nd)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    const unsigned two = Mma<T>::pack2(acc[pp][nd][r] * scale, acc[pp][nd][r + 1] * scale);
                    o[(size_t)c_row(r, h) * DH + 32 * nd + m] = (unsigned short)(two & 0xffffu);
                    o[(size_t)c_row(r + 1, h) * DH + 32 * nd + m] = (unsigned short)(two >> 16);
                }
        }
    }
}

template <int DH, int PB> constexpr size_t dq_ring_lds_bytes() {
    return 2 * (2 * 32 * DH * 2) + 4 * PB * 32 * DH * 2;  // K/V ring + d_out tiles of four waves
}

// PB is the direction block of the caller's choice (1, 2, 4, and 8 for head dim 64); head dim 128 has
// accumulation registers for four.
template <typename T, int DH, int PB, bool CAUSAL>
int launch_dq(const T* q, const T* k, const T* v, const T* g, const float* lse2, const float* o32, float* delta, T* dq,
               int n_bh, int H, int P, int T_len, float scale, hipStream_t stream) {
    constexpr int PBK = (DH == 128 && PB > 4) ? 4 : PB;
    const int n_qb = (T_len + 127) / 128;
    const int n_pb = (P + PBK - 1) / PBK;
    constexpr size_t lds_bytes = dq_ring_lds_bytes<DH, PBK>();
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");
    if (int rc = ensure_dynamic_lds<&dq_ring_kernel<T, DH, PBK, CAUSAL>>(lds_bytes)) return rc;
    hipLaunchKernelGGL((dq_ring_kernel<T, DH, PBK, CAUSAL>), dim3(grid_size(n_qb * n_pb, n_bh)), dim3(256), lds_bytes,
                       stream, q, k, v, g, lse2, o32, delta, dq, n_bh, H, P, T_len, scale);
    return LBI_OK;
}

}  // namespace attn_mfma
}  // namespace lbi
