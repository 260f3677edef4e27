// dK/dV kernel of the attention input-pullback, two (or, at head dim 64, four) directions per workgroup (fp16 /
// bf16 storage, head dim 64 or 128, two or more directions).
//
// A workgroup owns 128 keys and a pair of directions.  Its four waves are (kh, d): key half
// kh (64 keys), direction d.  The probabilities P = exp2(S c - lse2) do not depend on the
// direction, so each wave forms ONE 32 x 32 tile of S (keys 32 w .. 32 w + 31, w = wave id)
// and the packed, rounded P tile goes through LDS to the two waves that need it: per wave and
// step (32 queries) that is 2 KS products for S instead of 4 KS, and a quarter of the exp2 work.
//   S^T ...        S  = Q K_w^T                  A = Q tile (LDS), B = K_w tile (LDS, resident)
//   per wave (kh, d), its 64 keys x 32 queries:
//   dP - delta     = dO_d V^T - delta_d          A = dO_d tile (LDS), B = V (registers), C starts at -delta
//   dS             = P o (dP - delta)            P from the LDS exchange buffer
//   dV += P^T dO_d,   dK += dS^T Q               B through transpose reads of the streamed tiles
// S and P of step it+1 are formed during step it (its products sit between dV and dK, its
// vector work under the dK products), so one barrier per step publishes the next tile, the P
// tiles of the step and frees the stage of the step before.  Tiles (Q, dO_0, dO_1, row
// statistics) arrive by global_load_lds into a four-stage ring, three steps ahead.
// The vector work is slotted thinly between products, as in lbi_attn_dkdv128.h.
//
// DW = 2 (head dim 64, three directions or more): a wave takes a second direction (slots d and d + 2 of the
// workgroup's four), whose dP / dV / dK products run as a second part of the step on the same P tiles, V
// registers and Q tile; a stage then carries four d_out tiles.  At head dim 64 the accumulators of one direction
// fill half of the 256 accumulation registers and a step costs nearly the same whether it holds 28 products or 52,
// and the fixed cost of a key block (ring fill, first S / P tile, masked diagonal steps) is paid once for four
// directions: 2.39 -> 1.91 ms at B=8 H=12 T=1024 P=64, same results bit for bit.
#pragma once

#include <type_traits>

#include "lbi_attn_dkdv128.h"

namespace lbi {
namespace attn_mfma {

template <typename T, int DH, bool CAUSAL, int DW = 1>
__global__ __launch_bounds__(256) void dkdv_pair_kernel(const T* __restrict__ q, const T* __restrict__ k,
                                                      const T* __restrict__ v, const T* __restrict__ d_out,
                                                      const float* __restrict__ lse2, const float* __restrict__ delta,
                                                      T* __restrict__ dk, T* __restrict__ dv, int n_bh, int H, int P,
                                                      int T_len, float scale) {
    constexpr int KS = DH / 16, ND = DH / 32;
    constexpr int RB = DH * 2;                       // bytes per tile row
    constexpr int CPR = DH / 8;                      // 16-byte chunks per tile row
    constexpr int CPT = 32 * RB / 1024;              // 1 KiB wave-loads per tile: 8 (Dh 128) / 4 (Dh 64)
    // DW directions per wave (2 DW per workgroup).  Head dim 64 leaves half of the accumulation registers free, and
    // a step there is bound by what a tile costs whatever its products (the S / P tile, the exchange, the barrier, the
    // Q fragments), so with DW = 2 a wave runs the dP / dV / dK products of a second direction (direction slots d and
    // d + 2 of the workgroup's four) behind those of the first, on the same P tiles, V registers and Q tile.
    static_assert(DW == 1 || (DW == 2 && DH == 64), "accumulation registers: 2 DW x 64 x DH floats per lane group");
    constexpr int NTILE = 1 + 2 * DW;                // tiles per stage: Q, then one d_out tile per direction
    static_assert((NTILE * CPT) % 4 == 0, "tile wave-loads dealt evenly to four waves");
    constexpr int NXW = NTILE * CPT / 4;             // tile wave-loads per wave per stage: 6 / 3 (5 with DW = 2)
    constexpr unsigned TILE = 32 * RB;
    constexpr unsigned STATS = 4 * 512;              // per wave: 32 lse2, then two slots of 32 -delta floats
    constexpr unsigned STAGE = NTILE * TILE + STATS; // Q tile, d_out tiles, statistics
    constexpr int NDMA = NXW + 1;                    // global_load_lds per wave per stage
    constexpr int R = 4;
    constexpr unsigned KT0 = R * STAGE;              // K: four swizzled 32-key tiles
    constexpr unsigned PB0 = KT0 + 4 * TILE;         // two P exchange buffers: [tile w][kk][lane] x 16 bytes
    constexpr unsigned PBUF = 4 * 2 * 1024;
    extern __shared__ __align__(16) char smem[];

    const int n_kb = (T_len + 127) / 128;
    const int n_pp = (P + 2 * DW - 1) / (2 * DW);
    int bh, rem;
    if (!map_block(n_kb * n_pp, n_bh, bh, rem)) return;
    const int pp = rem / n_kb;
    const int kb = rem % n_kb;                       // ascending: longest key blocks first
    const int b = bh / H, hh = bh % H;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, m = lane & 31,
              h = lane >> 5;
    const int kh = wave >> 1, d = wave & 1;
    const int j0 = kb * 128;
    // the wave's directions: slots d (+ 2) of the workgroup's 2 DW; a surplus slot redoes the last direction and is
    // never stored
    const int p_first = 2 * DW * pp;
    bool active[DW];
    size_t prow_own[DW];
    const int j0w = min(j0 + 64 * kh, T_len - 64);   // this wave's 64 keys (dP, dV, dK)
    const int j0s = min(j0 + 32 * wave, T_len - 32); // this wave's S tile (equals j0w + 32 d inside the sequence)
    const size_t base = (size_t)bh * T_len * DH;
    const T* q_bh = q + base;
    const float* lse_bh = lse2 + (size_t)bh * T_len;
    size_t prow[2 * DW];
#pragma unroll
    for (int e = 0; e < 2 * DW; ++e) prow[e] = (((size_t)b * P + min(p_first + e, P - 1)) * H + hh) * T_len;
#pragma unroll
    for (int e = 0; e < DW; ++e) {
        active[e] = (j0 + 64 * kh < T_len) && (p_first + d + 2 * e < P);
        prow_own[e] = prow[d + 2 * e];
    }

    // ---- lane constants of the LDS addressing (see lbi_attn_dkdv128.h)
    const unsigned lane_nat = m * RB + ((h ^ swz<DH>(m)) << 4);
    const unsigned s16 = lane & 15, g1 = (lane >> 4) & 1;
    const unsigned tr_row = 4 * h + (s16 >> 2), tr_chunk = 2 * g1 + ((s16 & 3) >> 1);
    const unsigned lane_tr = tr_row * RB + ((tr_chunk ^ swz<DH>(tr_row)) << 4) + ((s16 & 1) << 3);
    const unsigned lane_stat = (unsigned)wave * 512 + 16 * h;  // + 32 g: lse2; + 128 slot + 32 g: -delta of that slot
    // statistics slots 1, 2: with DW = 1 the pair's two directions (the wave reads slot 1 + d), with DW = 2 the
    // wave's own two (slot 1 + e)
    auto nd_slot = [&](int e) __attribute__((always_inline)) { return DW == 1 ? 1 + d : 1 + e; };

    // ---- global -> LDS.  The NTILE CPT wave-loads of a stage are dealt round-robin: wave w takes
    // loads w, w + 4, ...; load c belongs to tile c / CPT and is its wave-load u = c % CPT.
    unsigned dma_off[NXW], dma_dst[NXW];   // lane offset inside the source tile; LDS offset inside a stage
    const T* dma_src[NXW];                 // wave-uniform source of each wave-load
#pragma unroll
    for (int x = 0; x < NXW; ++x) {
        const int c = wave + 4 * x;
        const int tile = c / CPT, u = c % CPT;
        const int sigma = 64 * u + lane;
        const int r = sigma / CPR;
        dma_off[x] = r * RB + (((sigma % CPR) ^ swz<DH>(r)) << 4);
        dma_dst[x] = tile * TILE + 1024 * u;
        dma_src[x] = tile == 0 ? q_bh : d_out + prow[tile - 1] * DH;
    }
    // lanes 0-7: lse2, 8-15: -delta of statistics slot 1, 16-23: of slot 2 (float4 each)
    const int slot_dir = DW == 1 ? (lane < 16 ? 0 : 1) : d + (lane < 16 ? 0 : 2);
    const float* stat_ptr = (lane < 8 ? lse_bh : delta + prow[slot_dir]) + 4 * (lane & 7);
    const unsigned lds0 = (unsigned)(size_t)(__attribute__((address_space(3))) char*)smem;
    auto issue_tile = [&](int i_row, unsigned stage_base) __attribute__((always_inline)) {
        const unsigned row_bytes = (unsigned)i_row * RB;
#pragma unroll
        for (int x = 0; x < NXW; ++x) dma16(dma_src[x], row_bytes + dma_off[x], lds0 + stage_base + dma_dst[x]);
        if (lane < 24) dma16_at(stat_ptr + i_row, lds0 + stage_base + NTILE * TILE + 512 * wave);
    };

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

    // ---- residents: V of the wave's 64 keys in registers; K of the workgroup's 128 keys in LDS
    u32x4 vf[2][KS];
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
            vf[t][ks] = *reinterpret_cast<const u32x4*>(v + base + (size_t)(j0w + 32 * t + m) * DH + 16 * ks + 8 * h);
    {
        char* kt_w = smem + KT0 + wave * TILE;       // wave w writes the tile it will read
#pragma unroll
        for (int u = 0; u < CPR / 2; ++u) {
            const int slot = 64 * u + lane;
            const int r = slot / CPR, c = slot % CPR;
            const u32x4 val = *reinterpret_cast<const u32x4*>(k + base + (size_t)(j0s + r) * DH + 8 * c);
            *reinterpret_cast<u32x4*>(kt_w + tile_off<DH>(r, c)) = val;
        }
    }
    const char* kt = smem + KT0 + wave * TILE;
    f32x16 acc_k[DW][2][ND], acc_v[DW][2][ND];
#pragma unroll
    for (int e = 0; e < DW; ++e)
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int nd = 0; nd < ND; ++nd) {
                acc_k[e][t][nd] = zero16();
                acc_v[e][t][nd] = zero16();
            }
    const float sc2 = scale * LOG2E;

    // P tile of this wave for the tile step in stage `sq`, written to exchange buffer `pbuf`.
    // thr: element 8g + e (query row) of the tile is above the diagonal iff 8g + e < thr.
    f32x16 s;
    f32x4 lq[4];
    auto p_quantum = [&](auto mask_tag, int g, int thr, u32x4 (&pw)[2]) __attribute__((always_inline)) {
        constexpr bool MASK = decltype(mask_tag)::value;
        pin_tile(s);
        float pr[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            pr[e] = __builtin_amdgcn_exp2f(s[4 * g + e] * sc2 - lq[g][e]);
            if (MASK && (8 * g + e < thr)) pr[e] = 0.0f;
        }
        unsigned w0 = Mma<T>::pack2(pr[0], pr[1]), w1 = Mma<T>::pack2(pr[2], pr[3]);
        pin_here(w0, w1);
        pw[g >> 1][2 * (g & 1)] = w0;
        pw[g >> 1][2 * (g & 1) + 1] = w1;
    };
    auto p_store = [&](unsigned pbuf, int kk, const u32x4& w) __attribute__((always_inline)) {
        *reinterpret_cast<u32x4*>(smem + pbuf + (2 * wave + kk) * 1024 + 16 * lane) = w;
    };

    const int i_begin = CAUSAL ? j0 : 0;
    const int n_it = (T_len - i_begin) / 32;
    const int n_pad = (n_it + R - 1) / R * R;
    const int head_end = CAUSAL ? min(4, n_pad) : 0;   // steps that can touch the diagonal (128 keys / 32)
    const int plain_end = head_end + (n_it > head_end ? (n_it - head_end) / R * R : 0);
    auto tile_row = [&](int it) __attribute__((always_inline)) { return min(i_begin + it * 32, T_len - 32); };
    // mask threshold of this wave's S tile at step it (padding steps mask everything)
    auto thr_of = [&](int it) __attribute__((always_inline)) {
        return it >= n_it ? (1 << 20) : CAUSAL ? j0s + m - 4 * h - (i_begin + it * 32) : -(1 << 20);
    };

    // First dO fragments (k-steps 0-2, slot ks % 3) and the -delta tile (accumulator layout) of the
    // step to come, fetched a step ahead so that a step starts with products, not with LDS latency.
    u32x4 ga[3];
    auto fetch_g = [&](const char* stage, int e, int ks) __attribute__((always_inline)) {
        if (ks < KS) ga[ks % 3] = lds16(stage + (1 + d + 2 * e) * TILE + (lane_nat ^ (ks << 5)));
    };
    f32x16 nd16;
    auto fetch_nd = [&](const char* stage, int e, int g) __attribute__((always_inline)) {
        const f32x4 d4 = lds_f4(stage + NTILE * TILE + lane_stat + 128 * nd_slot(e) + 32 * g);
#pragma unroll
        for (int e = 0; e < 4; ++e) nd16[4 * g + e] = d4[e];
    };

    // ---- prologue: tiles 0 .. R-2 requested; S / P of step 0 from tile 0
#pragma unroll
    for (int x = 0; x < R - 1; ++x) issue_tile(tile_row(x), x * STAGE);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm((R - 2) * NDMA));  // tile 0
    __syncthreads();                                          // also publishes the K tiles
    {
        u32x4 qa[KS], kf[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            qa[ks] = lds16(smem + (lane_nat ^ (ks << 5)));
            kf[ks] = lds16(kt + (lane_nat ^ (ks << 5)));
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            lq[g] = lds_f4(smem + NTILE * TILE + lane_stat + 32 * g);
            fetch_nd(smem, 0, g);
        }
        fetch_g(smem, 0, 0);
        fetch_g(smem, 0, 1);
        fetch_g(smem, 0, 2);
        s = Mma<T>::mma_v_start(qa[0], kf[0]);
#pragma unroll
        for (int ks = 1; ks < KS; ++ks) Mma<T>::mma_v(qa[ks], kf[ks], s);
        mma_v_settle(s);
        u32x4 pw[2];
        const int thr = thr_of(0);
#pragma unroll
        for (int g = 0; g < 4; ++g) p_quantum(std::true_type{}, g, thr, pw);
        p_store(PB0, 0, pw[0]);
        p_store(PB0, 1, pw[1]);
    }

    // One tile step.  SB: stage of the step, SN: of the next one (landed at the barrier), SR: the
    // stage freed by the barrier, refilled with tile refill_row.  PBC / PBN: P buffers of this
    // step and of the next.  thr_next: mask threshold of the P tile formed here (step it + 1).
    // The step is DW parts, one per direction of the wave: dP, dV, (part 0: S of the next step,) dK.  What a part
    // fetches "for the next" goes to the next part of this step or, from the last part, to part 0 of the next step.
    auto step = [&](auto mask_tag, auto sb_tag, auto sn_tag, auto sr_tag, auto pbc_tag, auto pbn_tag, int thr_next,
                    int refill_row) __attribute__((always_inline)) {
        constexpr unsigned SB = decltype(sb_tag)::value, SN = decltype(sn_tag)::value, SR = decltype(sr_tag)::value;
        constexpr unsigned PBC = decltype(pbc_tag)::value, PBN = decltype(pbn_tag)::value;
        const char* qt = smem + SB;
        const char* qn = smem + SN;

        // The barrier: this wave's share of tile it+1 has landed once all but the newest tile
        // load is done; everyone's P tiles of this step are written (LDS writes drained below).
        __builtin_amdgcn_s_waitcnt(waitcnt_vm((R - 3) * NDMA));
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");

        u32x4 pa[2][2];                   // P tiles of the wave's keys: from waves 2 kh and 2 kh + 1
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int kk = 0; kk < 2; ++kk)
                pa[t][kk] = lds16(smem + PBC + (2 * (2 * kh + t) + kk) * 1024 + 16 * lane);
        u32x4 qa[2], kf[2];               // operands of the next step's S, slot ks % 2
        auto fetch_s = [&](int ks) __attribute__((always_inline)) {
            if (ks < KS) {
                qa[ks % 2] = lds16(qn + (lane_nat ^ (ks << 5)));
                kf[ks % 2] = lds16(kt + (lane_nat ^ (ks << 5)));
            }
        };
        u32x4 pw[2];

        auto part = [&](auto e_tag) __attribute__((always_inline)) {
            constexpr int E = decltype(e_tag)::value;
            constexpr bool FIRST = E == 0, LAST = E == DW - 1;
            constexpr int NS = FIRST ? KS : 0;  // products of the S phase (one tile), part 0 only
            constexpr int NP = 2 * KS;        // products of the dP phase
            constexpr int NA = 4 * ND;        // products of the dV phase (and of the dK phase)
            constexpr int I_DV = NP, I_S = NP + NA, I_DK = NP + NA + NS, NPROD = NP + 2 * NA + NS;
            const char* gt = smem + SB + (1 + d + 2 * E) * TILE;
            const char* nxt = LAST ? qn : qt;   // stage and direction slot of the part after this one
            constexpr int NE = LAST ? 0 : E + 1;
            u32x4 bfr[3];  // tr fragment f of the dV (f < 2 ND: dO tile) and dK (Q tile) phases lives in slot f % 3
            auto fetch_tr = [&](int f) __attribute__((always_inline)) {
                if (f < 2 * ND) bfr[f % 3] = tr_frag(gt, f / ND, f % ND);
                else if (f < 4 * ND) bfr[f % 3] = tr_frag(qt, (f - 2 * ND) / ND, (f - 2 * ND) % ND);
            };
            f32x16 dp[2];
            u32x4 dsa[2][2];

            auto ds_quantum = [&](int qd) __attribute__((always_inline)) {
                const int g = qd >> 1, t = qd & 1;
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
            // Vector work and LDS traffic slotted after product i (0-based over the part).
            auto after = [&](int i) __attribute__((always_inline)) {
                __builtin_amdgcn_sched_barrier(0);
                // dP operands: pair ks = i / 2 consumed at odd i < NP; refill its slot
                if (i < NP && (i & 1)) fetch_g(qt, E, i / 2 + 3);
                if (FIRST && i == 1) issue_tile(refill_row, SR);  // the stage freed by the barrier
                if (i == I_DK + 2) fetch_g(nxt, NE, 0);       // the next part's first dO fragments
                if (i == I_DK + 4) fetch_g(nxt, NE, 1);
                if (i == I_DK + 6) fetch_g(nxt, NE, 2);
                // tr fragments: three fetched ahead of the dV phase, then one per consumed fragment
                if (i == NP - 6) fetch_tr(0);
                if (i == NP - 4) fetch_tr(1);
                if (i == NP - 2) fetch_tr(2);
                if (i >= I_DV && i < I_S && ((i - I_DV) & 1)) fetch_tr((i - I_DV) / 2 + 3);
                if (i >= I_DK && ((i - I_DK) & 1)) fetch_tr(2 * ND + (i - I_DK) / 2 + 3);
                // next step's S operands: three ahead of the S phase, then one per product; its statistics
                if (FIRST) {
                    if (i == I_S - 4) fetch_s(0);
                    if (i == I_S - 2) fetch_s(1);
                    if (i >= I_S && i < I_DK) fetch_s(i - I_S + 2);
                }
                // dS quanta: eight between the end of dP and the start of dK (rows 0-15 first)
                constexpr int ds_first = NP + 2, ds_span = I_DK - 3 - ds_first;
#pragma unroll
                for (int qd = 0; qd < 8; ++qd)
                    if (i == ds_first + (qd * ds_span) / 7) ds_quantum(qd);
                // P quanta of the next step: four under the dK products of part 0, then the exchange buffer
                if (FIRST) {
                    constexpr int p_first_i = I_DK + 1, p_span = NA - 5;
#pragma unroll
                    for (int g = 0; g < 4; ++g)   // its row statistics, two products ahead
                        if (i == p_first_i + (g * p_span) / 3 - 2) lq[g] = lds_f4(qn + NTILE * TILE + lane_stat + 32 * g);
#pragma unroll
                    for (int g = 0; g < 4; ++g)
                        if (i == p_first_i + (g * p_span) / 3) {
                            if (g == 0) mma_v_settle(s);
                            p_quantum(mask_tag, g, thr_next, pw);
                            if (g == 1) p_store(PBN, 0, pw[0]);
                            if (g == 3) p_store(PBN, 1, pw[1]);
                        }
                }
                // -delta tile of the next part
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    if (i == NPROD - 5 + g) fetch_nd(nxt, NE, g);
                __builtin_amdgcn_sched_barrier(0);
            };

            // ---- dP - delta = dO V^T - delta
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                if (ks == 0) dp[0] = Mma<T>::mma_v_c(ga[0], vf[0][0], nd16);
                else Mma<T>::mma_v(ga[ks % 3], vf[0][ks], dp[0]);
                after(2 * ks);
                if (ks == 0) dp[1] = Mma<T>::mma_v_c(ga[0], vf[1][0], nd16);
                else Mma<T>::mma_v(ga[ks % 3], vf[1][ks], dp[1]);
                after(2 * ks + 1);
            }
            // ---- dV += P^T dO
#pragma unroll
            for (int f = 0; f < 2 * ND; ++f) {
                const int kk = f / ND, nd = f % ND;
                acc_v[E][0][nd] = Mma<T>::mma(pa[0][kk], bfr[f % 3], acc_v[E][0][nd]);
                after(I_DV + 2 * f);
                acc_v[E][1][nd] = Mma<T>::mma(pa[1][kk], bfr[f % 3], acc_v[E][1][nd]);
                after(I_DV + 2 * f + 1);
            }
            // ---- S of the next step (this wave's tile)
            if (FIRST) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (ks == 0) s = Mma<T>::mma_v_start(qa[0], kf[0]);
                    else Mma<T>::mma_v(qa[ks % 2], kf[ks % 2], s);
                    after(I_S + ks);
                }
            }
            // ---- dK += dS^T Q
#pragma unroll
            for (int f = 2 * ND; f < 4 * ND; ++f) {
                const int kk = (f - 2 * ND) / ND, nd = f % ND;
                acc_k[E][0][nd] = Mma<T>::mma(dsa[0][kk], bfr[f % 3], acc_k[E][0][nd]);
                after(I_DK + 2 * (f - 2 * ND));
                acc_k[E][1][nd] = Mma<T>::mma(dsa[1][kk], bfr[f % 3], acc_k[E][1][nd]);
                after(I_DK + 2 * (f - 2 * ND) + 1);
            }
        };
        part(std::integral_constant<int, 0>{});
        if constexpr (DW == 2) part(std::integral_constant<int, 1>{});
    };

    auto one_step = [&](auto mask_tag, auto slot_tag, int it) __attribute__((always_inline)) {
        constexpr int SLOT = decltype(slot_tag)::value;
        step(mask_tag, std::integral_constant<unsigned, SLOT * STAGE>{},
             std::integral_constant<unsigned, ((SLOT + 1) % R) * STAGE>{},
             std::integral_constant<unsigned, ((SLOT + R - 1) % R) * STAGE>{},
             std::integral_constant<unsigned, PB0 + (SLOT & 1) * PBUF>{},
             std::integral_constant<unsigned, PB0 + ((SLOT + 1) & 1) * PBUF>{}, thr_of(it + 1), tile_row(it + R - 1));
    };
    auto group = [&](auto mask_tag, int it0) __attribute__((always_inline)) {
        one_step(mask_tag, std::integral_constant<int, 0>{}, it0);
        one_step(mask_tag, std::integral_constant<int, 1>{}, it0 + 1);
        one_step(mask_tag, std::integral_constant<int, 2>{}, it0 + 2);
        one_step(mask_tag, std::integral_constant<int, 3>{}, it0 + 3);
    };
    // The masked variant is needed where the P tile formed in a step (that of the step after)
    // can touch the diagonal or belongs to a padding step.
    int it = 0;
    for (; it < head_end; it += R) group(std::true_type{}, it);
    for (; it < plain_end; it += R) group(std::false_type{}, it);
    for (; it < n_pad; it += R) group(std::true_type{}, it);
    __builtin_amdgcn_s_waitcnt(waitcnt_vm(0));

#pragma unroll
    for (int e = 0; e < DW; ++e) {
        if (!active[e]) continue;
        unsigned short* ok = reinterpret_cast<unsigned short*>(dk + (prow_own[e] + j0w) * DH);
        unsigned short* ov = reinterpret_cast<unsigned short*>(dv + (prow_own[e] + j0w) * DH);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int nd = 0; nd < ND; ++nd)
#pragma unroll
                for (int r = 0; r < 16; r += 2) {
                    const unsigned k2 = Mma<T>::pack2(acc_k[e][t][nd][r] * scale, acc_k[e][t][nd][r + 1] * scale);
                    const unsigned v2 = Mma<T>::pack2(acc_v[e][t][nd][r], acc_v[e][t][nd][r + 1]);
                    const size_t o0 = (size_t)(32 * t + c_row(r, h)) * DH + 32 * nd + m;
                    const size_t o1 = (size_t)(32 * t + c_row(r + 1, h)) * DH + 32 * nd + m;
                    ok[o0] = (unsigned short)(k2 & 0xffffu);
                    ok[o1] = (unsigned short)(k2 >> 16);
                    ov[o0] = (unsigned short)(v2 & 0xffffu);
                    ov[o1] = (unsigned short)(v2 >> 16);
                }
    }
}

template <int DH, int DW = 1> constexpr size_t dkdv_pair_lds_bytes() {
    // 4 stages (Q tile, 2 DW d_out tiles, statistics) + K of 128 keys + 2 P buffers
    return 4 * ((1 + 2 * DW) * 32 * DH * 2 + 4 * 512) + 4 * 32 * DH * 2 + 2 * 8 * 1024;
}

template <typename T, int DH, bool CAUSAL, int DW>
int launch_dkdv_pair_as(const T* q, const T* k, const T* v, const T* g, const float* lse2, const float* delta, T* dk,
                        T* dv, int n_bh, int H, int P, int T_len, float scale, hipStream_t stream) {
    const int n_kb = (T_len + 127) / 128;
    const int n_pp = (P + 2 * DW - 1) / (2 * DW);
    constexpr size_t lds_bytes = dkdv_pair_lds_bytes<DH, DW>();
    static_assert(lds_bytes <= 160 * 1024, "LDS budget");
    if (int rc = ensure_dynamic_lds<&dkdv_pair_kernel<T, DH, CAUSAL, DW>>(lds_bytes)) return rc;
    hipLaunchKernelGGL((dkdv_pair_kernel<T, DH, CAUSAL, DW>), dim3(grid_size(n_kb * n_pp, n_bh)), dim3(256), lds_bytes,
                       stream, q, k, v, g, lse2, delta, dk, dv, n_bh, H, P, T_len, scale);
    return LBI_OK;
}

// Head dim 64 with three directions or more: two directions per wave (four per workgroup).
template <typename T, int DH, bool CAUSAL>
int launch_dkdv_pair(const T* q, const T* k, const T* v, const T* g, const float* lse2, const float* delta, T* dk,
                      T* dv, int n_bh, int H, int P, int T_len, float scale, hipStream_t stream) {
    if constexpr (DH == 64) {
        if (P >= 3)
            return launch_dkdv_pair_as<T, DH, CAUSAL, 2>(q, k, v, g, lse2, delta, dk, dv, n_bh, H, P, T_len, scale, stream);
    }
    return launch_dkdv_pair_as<T, DH, CAUSAL, 1>(q, k, v, g, lse2, delta, dk, dv, n_bh, H, P, T_len, scale, stream);
}

}  // namespace attn_mfma
}  // namespace lbi
