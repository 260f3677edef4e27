// dK/dV kernel of the attention input-pullback (fp16 / bf16 storage, head dim 64 or 128).
//
// Same ownership and arithmetic as attn_mfma::dkdv_kernel (one wave = 64 keys x one
// direction, workgroup = 256 keys, Q and d_out_p streamed in 32-query tiles), with the
// data path rebuilt around what the counters showed: the first version spent as many
// cycles in VALU work and in waits as in MFMA.
//
//  * Q / d_out tiles and the lse2 / delta rows go global -> LDS with global_load_lds
//    (16 bytes per lane, no staging registers, no ds_write), three tiles ahead, into a
//    four-stage ring (a tile load takes longer than a step).  The loop is unrolled by
//    four so the stage is a compile-time immediate of every LDS read.
//  * The XOR swizzle is linear over GF(2), so every LDS address is
//    (lane constant) ^ (compile-time constant) + immediate: one VALU op per read at most.
//  * Causal masking runs only in the first 8 steps of a workgroup (queries that
//    are not past all of its 256 keys); the main loop has no compare / select.
//  * The products are ordered S, dP, [P], dV, [dS], dK so the VALU phase in brackets
//    has independent MFMA work on either side to overlap with.
#pragma once

#include <type_traits>

#include "lbi_attn_mfma.h"

namespace lbi {
namespace attn_mfma {

// s_waitcnt immediate with only vmcnt constrained (gfx9 encoding: vmcnt = [15:14|3:0],
// expcnt [6:4], lgkmcnt [11:8]).
constexpr int waitcnt_vm(int n) { return (n & 15) | ((n >> 4) << 14) | (7 << 4) | (15 << 8); }

// 64 lanes x 16 bytes, global -> LDS.  Lane l reads 16 bytes at base + voff(l) and the
// data lands at lds_base + 16*l.  lds_base must be wave-uniform.
__device__ __forceinline__ void dma16(const void* base, unsigned voff, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(voff), "s"(base)
                 : "memory");
}

// The same with a full 64-bit address per lane (no common base).
__device__ __forceinline__ void dma16_at(const void* lane_ptr, unsigned lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                 :
                 : "s"(__builtin_amdgcn_readfirstlane(lds_base)), "v"(lane_ptr)
                 : "memory");
}

template <typename T, int DH, bool CAUSAL>
__global__ __launch_bounds__(256) void dkdv_ring_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                      const T* __restrict__ v, const T* __restrict__ d_out,
                                                      const float* __restrict__ lse2, const float* __restrict__ delta,
                                                      T* __restrict__ dk, T* __restrict__ dv, int n_bh, int H, int P,
                                                      int T_len, float scale) {
    constexpr int KS = DH / 16, ND = DH / 32;
    constexpr int RB = DH * 2;                     // bytes per tile row
    constexpr int CPR = DH / 8;                    // 16-byte chunks per tile row
    constexpr int NX = DH / 64;                    // global_load_lds per tile per wave
    constexpr unsigned TILE = 32 * RB;             // 8 KiB (Dh 128) / 4 KiB (Dh 64)
    constexpr unsigned STATS = 4 * 256;            // per wave: 32 lse2 + 32 delta floats
    constexpr unsigned STAGE = 2 * TILE + STATS;   // Q tile, d_out tile, stats
    constexpr int NDMA = 2 * NX + 1;               // global_load_lds per wave per tile step
    constexpr int R = 4;                           // ring stages
    extern __shared__ __align__(16) char smem[];   // [R][STAGE], then V

    const int n_kb = (T_len + 255) / 256;
    int bh, rem;
    if (!map_block(n_kb * P, n_bh, bh, rem)) return;
    const int p = rem / n_kb;
    const int kb = rem % n_kb;
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, m = lane & 31, h = lane >> 5;
    const bool active = kb * 256 + wave * 64 < T_len;
    const int j0w = min(kb * 256 + wave * 64, T_len - 64);
    const size_t base = (size_t)bh * T_len * DH;
    const size_t prow = (((size_t)b * P + p) * H + hh) * T_len;
    const T* q_bh = q + base;
    const T* g_p = d_out + prow * DH;
    const float* lse_bh = lse2 + (size_t)bh * T_len;
    const float* delta_p = delta + prow;

    // ---- lane constants of the LDS addressing -------------------------------------------
    // nat: tile_off(m, 2ks + h) == lane_nat ^ (ks << 5).  tr: the address of the transpose read for
    // (k0, hi, nd) is (lane_tr ^ (nd << 6 | hi << 5)) + (k0 + 8 hi) * RB; both follow from the
    // swizzle being an XOR of row bits into chunk bits.
    const unsigned lane_nat = m * RB + ((h ^ swz<DH>(m)) << 4);
    const unsigned s16 = lane & 15, g1 = (lane >> 4) & 1;
    const unsigned tr_row = 4 * h + (s16 >> 2), tr_chunk = 2 * g1 + ((s16 & 3) >> 1);
    const unsigned lane_tr = tr_row * RB + ((tr_chunk ^ swz<DH>(tr_row)) << 4) + ((s16 & 1) << 3);
    const unsigned lane_stat = (unsigned)wave * 256 + 16 * h;  // + 32*g (lse2), + 128 (delta)

    // ---- global -> LDS: this wave's share of a tile step ---------------------------------
    // Tile slot sigma = 64u + lane (u = NX*wave + x): row sigma/CPR, physical chunk sigma%CPR.
    unsigned dma_off[NX];
#pragma unroll
    for (int x = 0; x < NX; ++x) {
        const int sigma = 64 * (NX * wave + x) + lane;
        const int r = sigma / CPR;
        dma_off[x] = r * RB + (((sigma % CPR) ^ swz<DH>(r)) << 4);
    }
    // lanes 0-7: lse2 float4 #lane, lanes 8-15: delta float4 #(lane-8); the two arrays need not
    // share an allocation, so each lane carries its own 64-bit address
    const float* stat_ptr = (lane < 8 ? lse_bh : delta_p) + 4 * (lane & 7);
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem;
    auto issue_tile = [&](int i_row, unsigned stage_base) __attribute__((always_inline)) {
        const unsigned row_bytes = (unsigned)i_row * RB;
#pragma unroll
        for (int x = 0; x < NX; ++x) {
            dma16(q_bh, row_bytes + dma_off[x], lds0 + stage_base + 1024 * (NX * wave + x));
            dma16(g_p, row_bytes + dma_off[x], lds0 + stage_base + TILE + 1024 * (NX * wave + x));
        }
        // Every wave keeps its own copy of the 64 row statistics: no cross-wave dependency.
        if (lane < 16) dma16_at(stat_ptr + i_row, lds0 + stage_base + 2 * TILE + 256 * wave);
    };

    // K of this wave's 64 keys stays in registers (B operand of S).  V of the same keys sits
    // in LDS behind the two stages, as two swizzled 32-row tiles per wave: registers hold
    // the 256 accumulators, K, and the S / dP tiles of a step, and no more.
    u32x4 kf[2][KS];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            kf[t][ks] = *reinterpret_cast<const u32x4*>(k + base + (size_t)(j0w + 32 * t + m) * DH + 16 * ks + 8 * h);
    {
        char* vt_w = smem + R * STAGE + wave * 2 * TILE;
#pragma unroll
        for (int u = 0; u < CPR; ++u) {
            const int slot = 64 * u + lane;  // 16-byte slot of the wave's 64-row block
            const int r = slot / CPR, c = slot % CPR;
            const u32x4 val = *reinterpret_cast<const u32x4*>(v + base + (size_t)(j0w + r) * DH + 8 * c);
            *reinterpret_cast<u32x4*>(vt_w + (r >> 5) * TILE + tile_off<DH>(r & 31, c)) = val;
        }
    }
    const char* vt = smem + R * STAGE + wave * 2 * TILE;
    f32x16 acc_k[2][ND], acc_v[2][ND];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int nd = 0; nd < ND; ++nd) {
            acc_k[t][nd] = zero16();
            acc_v[t][nd] = zero16();
        }
    const float sc2 = scale * LOG2E;

    auto lds16 = [&](const char* p) __attribute__((always_inline)) {
        return *reinterpret_cast<const u32x4*>(p);
    };
    auto lds_f4 = [&](const char* p) __attribute__((always_inline)) {
        return *reinterpret_cast<const f32x4*>(p);
    };
    auto tr_frag = [&](const char* tile, int kk, int nd) __attribute__((always_inline)) {
        typedef __attribute__((address_space(3))) s16x4* lds_ptr;
        const s16x4 lo =
            __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_ptr)(tile + (lane_tr ^ (nd << 6)) + (16 * kk) * RB));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_ptr)(tile + (lane_tr ^ ((nd << 6) | 32)) + (16 * kk + 8) * RB));
        const u32x2 l2 = __builtin_bit_cast(u32x2, lo), h2 = __builtin_bit_cast(u32x2, hi);
        return u32x4{l2[0], l2[1], h2[0], h2[1]};
    };

    // One tile step on the stage at byte offset SB: 8 KS matrix products in four phases,
    //   S = Q K^T   dP = dO V^T - delta   dV += P^T dO   dK += dS^T Q        (2 KS, 2 KS, 4 ND, 4 ND products)
    // and sixteen "quanta" of vector work, one per (g, t) block of four rows of a 32 x 32 tile:
    //   P quantum:  exp2(S c - lse2), mask, round, pack        dS quantum:  P o dP, round, pack
    // The matrix pipe overlaps vector instructions of the same wave only while few of them sit
    // between two products, so the quanta are spread thinly over the products that do not
    // need their results yet instead of being bunched behind the phase that feeds them:
    //   P quanta 0-3 (rows 0-15: the k-step 0 operands of dV) under the dP products, 4-7 under
    //   the first half of dV; dS quanta 0-3 under the second half of dV, 4-7 under the first
    //   half of dK.  LDS operands are fetched two product pairs ahead of their use.
    // thr: element (t, 8g+e) is above the diagonal iff 8g + e < thr + 32t.
    // Operands of the S phase and the row statistics of the step to come: fetched during the
    // dK phase of the step before (the first ones ahead of the loop), so a step starts with
    // its products, not with LDS latency.
    u32x4 qa[KS];
    f32x4 lq[4];      // lse2 of rows 8g + 4h .. + 3
    f32x16 nd16;      // -delta of the same rows, laid out as an accumulator tile
    auto fetch_q = [&](const char* stage, int ks) __attribute__((always_inline)) {
        qa[ks] = lds16(stage + (lane_nat ^ (ks << 5)));
    };
    auto fetch_stats = [&](const char* stage, int g) __attribute__((always_inline)) {
        lq[g] = lds_f4(stage + 2 * TILE + lane_stat + 32 * g);
        const f32x4 d4 = lds_f4(stage + 2 * TILE + lane_stat + 128 + 32 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) nd16[4 * g + e] = d4[e];
    };

    auto step = [&](auto mask_tag, auto stage_tag, auto next_tag, auto refill_tag, int thr, int refill_row)
                    __attribute__((always_inline)) {
        constexpr bool MASK = decltype(mask_tag)::value;
        constexpr unsigned SB = decltype(stage_tag)::value;
        constexpr unsigned SN = decltype(next_tag)::value;      // stage of the next tile
        constexpr unsigned SR = decltype(refill_tag)::value;    // stage of the tile before: free after the mid-step barrier
        constexpr int NS = 2 * KS;      // products of the S phase (and of the dP phase)
        constexpr int NA = 4 * ND;      // products of the dV phase (and of the dK phase)
        constexpr int NPROD = 2 * NS + 2 * NA;
        const char* qt = smem + SB;
        const char* gt = smem + SB + TILE;
        const char* st = smem + SB + 2 * TILE;

        u32x4 ga[3], va[3], vb[3];  // dP operands of k-step ks live in slot ks % 3
        auto fetch_dp = [&](int ks) __attribute__((always_inline)) {
            ga[ks % 3] = lds16(gt + (lane_nat ^ (ks << 5)));
            va[ks % 3] = lds16(vt + (lane_nat ^ (ks << 5)));
            vb[ks % 3] = lds16(vt + TILE + (lane_nat ^ (ks << 5)));
        };
        u32x4 bfr[3];  // tr fragment f of the dV (f < 2 ND: d_out tile) and dK (Q tile) phases lives in slot f % 3
        auto fetch_tr = [&](int f) __attribute__((always_inline)) {
            if (f < 2 * ND) bfr[f % 3] = tr_frag(gt, f / ND, f % ND);
            else if (f < 4 * ND) bfr[f % 3] = tr_frag(qt, (f - 2 * ND) / ND, (f - 2 * ND) % ND);
        };
        f32x16 s[2], dp[2];
        u32x4 pa[2][2], dsa[2][2];

        auto p_quantum = [&](int q) __attribute__((always_inline)) {
            const int g = q >> 1, t = q & 1;
            pin_tile(s[t]);
            float pr[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                pr[e] = __builtin_amdgcn_exp2f(s[t][4 * g + e] * sc2 - lq[g][e]);
                if (MASK && (8 * g + e < thr + 32 * t)) pr[e] = 0.0f;
            }
            unsigned w0 = Mma<T>::pack2(pr[0], pr[1]), w1 = Mma<T>::pack2(pr[2], pr[3]);
            pin_here(w0, w1);
            pa[t][g >> 1][2 * (g & 1)] = w0;
            pa[t][g >> 1][2 * (g & 1) + 1] = w1;
        };
        auto ds_quantum = [&](int q) __attribute__((always_inline)) {
            const int g = q >> 1, t = q & 1;
            pin_tile(dp[t]);
            const unsigned p0 = pa[t][g >> 1][2 * (g & 1)], p1 = pa[t][g >> 1][2 * (g & 1) + 1];
            const float d0 = Mma<T>::lo(p0) * dp[t][4 * g + 0];  // dp already holds dP - delta
            const float d1 = Mma<T>::hi(p0) * dp[t][4 * g + 1];
            const float d2 = Mma<T>::lo(p1) * dp[t][4 * g + 2];
            const float d3 = Mma<T>::hi(p1) * dp[t][4 * g + 3];
            unsigned w0 = Mma<T>::pack2(d0, d1), w1 = Mma<T>::pack2(d2, d3);
            pin_here(w0, w1);
            dsa[t][g >> 1][2 * (g & 1)] = w0;
            dsa[t][g >> 1][2 * (g & 1) + 1] = w1;
        };
        // Vector work and LDS fetches slotted after product i (0-based over the whole step).
        auto after = [&](int i) __attribute__((always_inline)) {
            __builtin_amdgcn_sched_barrier(0);  // nothing moves across a product: the slotting below is the schedule
            // ---- fetches
            if (i == NS / 2) fetch_dp(0);
            if (i == NS / 2 + 2) fetch_dp(1);
            if (i == NS - 2) fetch_dp(2);
            if (i >= NS && i < 2 * NS && (i & 1)) {            // pair ks = (i - NS) / 2 consumed: refill its slot
                const int ks = (i - NS) / 2;
                if (ks + 3 < KS) fetch_dp(ks + 3);
            }
            if (i == 2 * NS - 6) fetch_tr(0);
            if (i == 2 * NS - 4) fetch_tr(1);
            if (i == 2 * NS - 2) fetch_tr(2);
            if (i >= 2 * NS && (i & 1)) fetch_tr((i - 2 * NS) / 2 + 3);  // fragment (i - 2NS)/2 consumed
            if (i == 2 * NS - 1) {
                // Half way: this wave's share of the next tile has landed once all but the newest
                // tile load is done; the barrier publishes everyone's share and tells that every wave
                // is done with the tile before this one, whose stage is refilled.  (No LDS wait: the
                // reads in flight belong to stages that stay as they are.)
                __builtin_amdgcn_s_waitcnt(waitcnt_vm((R - 3) * NDMA));
                __builtin_amdgcn_s_barrier();
                issue_tile(refill_row, SR);
            }
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                if (i == 2 * NS + NA + 2 * ks) fetch_q(smem + SN, ks);
#pragma unroll
            for (int g = 0; g < 4; ++g)
                if (i == 2 * NS + NA + 1 + 2 * g) fetch_stats(smem + SN, g);
            // ---- quanta.  Sixteen quanta over the products NS+1 .. NPROD-NA/2-2, evenly.
            constexpr int first = NS + 1, span = NPROD - NA / 2 - 2 - first;
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                if (i == first + (q * span) / 15) {
                    if (q == 0) mma_v_settle(s[0], s[1]);
                    if (q < 8) p_quantum(q);
                    else ds_quantum(q - 8);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        };

        // ---- S = Q K^T
        s[0] = Mma<T>::mma_v_start(qa[0], kf[0][0]);
        after(0);
        s[1] = Mma<T>::mma_v_start(qa[0], kf[1][0]);
        after(1);
#pragma unroll
        for (int ks = 1; ks < KS; ++ks) {
            Mma<T>::mma_v(qa[ks], kf[0][ks], s[0]);
            after(2 * ks);
            Mma<T>::mma_v(qa[ks], kf[1][ks], s[1]);
            after(2 * ks + 1);
        }
        // ---- dP - delta = dO V^T - delta
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            if (ks == 0) dp[0] = Mma<T>::mma_v_c(ga[0], va[0], nd16);
            else Mma<T>::mma_v(ga[ks % 3], va[ks % 3], dp[0]);
            after(NS + 2 * ks);
            if (ks == 0) dp[1] = Mma<T>::mma_v_c(ga[0], vb[0], nd16);
            else Mma<T>::mma_v(ga[ks % 3], vb[ks % 3], dp[1]);
            after(NS + 2 * ks + 1);
        }
        // ---- dV += P^T dO, then dK += dS^T Q
#pragma unroll
        for (int f = 0; f < 4 * ND; ++f) {
            const int ff = f % (2 * ND), kk = ff / ND, nd = ff % ND;
            if (f < 2 * ND) {
                acc_v[0][nd] = Mma<T>::mma(pa[0][kk], bfr[f % 3], acc_v[0][nd]);
                after(2 * NS + 2 * f);
                acc_v[1][nd] = Mma<T>::mma(pa[1][kk], bfr[f % 3], acc_v[1][nd]);
                after(2 * NS + 2 * f + 1);
            } else {
                acc_k[0][nd] = Mma<T>::mma(dsa[0][kk], bfr[f % 3], acc_k[0][nd]);
                after(2 * NS + 2 * f);
                acc_k[1][nd] = Mma<T>::mma(dsa[1][kk], bfr[f % 3], acc_k[1][nd]);
                after(2 * NS + 2 * f + 1);
            }
        }
    };

    // ---- tile loop: a ring of R stages; tile it + R - 1 is requested half way through step it.
    // A group is R consecutive steps, so every stage offset is an immediate.  Steps past the end of the sequence
    // (the group count is rounded up) run on a re-read tile with everything masked.
    const int i_begin = CAUSAL ? kb * 256 : 0;
    const int n_it = (T_len - i_begin) / 32;
    const int n_pad = (n_it + R - 1) / R * R;
    const int head_end = CAUSAL ? min(8, n_pad) : 0;  // steps that can touch the diagonal (8 = 256 keys / 32)
    const int plain_end = head_end + (n_it > head_end ? (n_it - head_end) / R * R : 0);
    auto tile_row = [&](int it) __attribute__((always_inline)) { return min(i_begin + it * 32, T_len - 32); };
#pragma unroll
    for (int x = 0; x < R - 1; ++x) issue_tile(tile_row(x), x * STAGE);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm((R - 2) * NDMA));  // tile 0
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) fetch_q(smem, ks);
#pragma unroll
    for (int g = 0; g < 4; ++g) fetch_stats(smem, g);
    auto one_step = [&](auto mask_tag, auto slot_tag, int it) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_tag)::value;
        // real steps of the non-causal case mask nothing; padding steps mask everything
        const int thr = it >= n_it ? (1 << 20) : CAUSAL ? j0w + m - 4 * h - (i_begin + it * 32) : -(1 << 20);
        step(mask_tag, std::integral_constant<unsigned, SLOT * STAGE>{},
             std::integral_constant<unsigned, ((SLOT + 1) % R) * STAGE>{},
             std::integral_constant<unsigned, ((SLOT + R - 1) % R) * STAGE>{}, thr, tile_row(it + R - 1));
    };
    auto group = [&](auto mask_tag, int it0) __attribute__((always_inline)) {
        one_step(mask_tag, std::integral_constant<int, 0>{}, it0);
        one_step(mask_tag, std::integral_constant<int, 1>{}, it0 + 1);
        one_step(mask_tag, std::integral_constant<int, 2>{}, it0 + 2);
        one_step(mask_tag, std::integral_constant<int, 3>{}, it0 + 3);
    };
    int it = 0;
    for (; it < head_end; it += R) group(std::true_type{}, it);
    for (; it < plain_end; it += R) group(std::false_type{}, it);
    for (; it < n_pad; it += R) group(std::true_type{}, it);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));

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

template <int DH> constexpr size_t dkdv_ring_lds_bytes() {
    return 4 * (2 * 32 * DH * 2 + 4 * 256) + 4 * 2 * 32 * DH * 2;  // 4 stages + V of 256 keys
}

template <typename T, int DH, bool CAUSAL>
int launch_dkdv(const T* q, const T* k, const T* v, const T* g, const float* lse2, const float* delta, T* dk, T* dv,
                 int n_bh, int H, int P, int T_len, float scale, hipStream_t stream) {
    const int n_kb = (T_len + 255) / 256;
    constexpr size_t lds_bytes = dkdv_ring_lds_bytes<DH>();
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");
    if (int rc = ensure_dynamic_lds<&dkdv_ring_kernel<T, DH, CAUSAL>>(lds_bytes)) return rc;
    hipLaunchKernelGGL((dkdv_ring_kernel<T, DH, CAUSAL>), dim3(grid_size(n_kb * P, n_bh)), dim3(256), lds_bytes, stream,
                       q, k, v, g, lse2, delta, dk, dv, n_bh, H, P, T_len, scale);
    return LBI_OK;
}

}  // namespace attn_mfma
}  // namespace lbi
