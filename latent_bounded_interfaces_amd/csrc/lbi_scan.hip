// Suffix scan of interface pullback matrices for gfx950 (MI355X).
//
//   out[b, r] = mats[b, r] @ out[b, r+1],  out[b, K] = I          (matrices)
//   out[b, r] = mats[b, r] @ out[b, r+1],  out[b, K] = g[b]       (cotangents)
//
// The product is a LEFT multiplication, so column blocks of the running suffix
// are independent: a workgroup owns `CB` columns of one batch element, keeps
// that d x CB block on chip, streams mats[b, K-1] ... mats[b, 0] from HBM once
// and writes every suffix block as it goes.  This does K-1 products per batch
// element (the log-depth scan of the reference, cuda/interface/suffix_scan.cu:89-108,
// does sum_l (K - 2^l)), needs no synchronisation between workgroups, and sums
// in a fixed order, so reruns are bit-identical.
#include "lbi_common.h"

#include <cstdlib>
#include <initializer_list>
#include <type_traits>

#include "lbi_scan_colsplit.h"
#include "lbi_scan_split.h"

namespace lbi {
namespace {

// ---------------------------------------------------------------------------------------
// MFMA path: d in {32, 64, 128, 256}.
//
// One wave computes an RT x CB tile of the new suffix block with
// v_mfma_f32_32x32x2_f32.  Operand layout of that instruction (lane = 32*h + m):
//   A (32 x 2):  lane holds A[m][h]        B (2 x 32):  lane holds B[h][m]
//   C (32 x 32): register i of the lane holds C[8*(i/4) + 4*h + i%4][m]
// Which actual k index feeds slot h of which instruction is free as long as A and
// B agree, so a lane loads 16 CONSECUTIVE k of its row (64 bytes; the h=0 and h=1
// lanes of a row together cover one 128-byte line) and uses them for 16
// instructions.  The matching B values, S[k][col] for 16 consecutive k and the
// lane's column, are contiguous because the block is kept TRANSPOSED in LDS
// (St[col][k], row pitch D+4 floats so 16-byte reads of 16 lanes hit 64 distinct
// banks).  The C layout gives each lane 4 consecutive rows of one column, which is
// one 16-byte write into St for the next step.
//
// A rows are private to a wave, so mats go global -> registers directly,
// prefetched one 32-wide k chunk ahead, across step boundaries too (mats do not
// depend on the running product).  St is double buffered: one barrier per step.
// ---------------------------------------------------------------------------------------
//
// COT: the kernel also runs the cotangent chain v[r] = mats[r] @ v[r+1], v[K] = g.  The
// fragments of mats[r] that feed the MFMAs are already in registers, so a step costs
// D/2 extra FMAs per lane (and nothing from HBM); every column block computes the chain,
// block 0 writes it.
// Which part of the chain a workgroup runs.  `phase` 0 is the whole chain of a batch element (K - 1 dependent
// steps).  Phases 1-3 are the K-parallel form for batches too small to fill the chip with one chain per column
// block: the chain is cut into C chunks; chunk c >= 1 starts at matrix b_c = cL - s and has L matrices (the last
// one what is left), chunk 0 has the first L - s (s = 1: every chunk then has L - 1 steps in phase 3, where chunk 0,
// which has no boundary product of its own to skip, would otherwise run one step longer than the rest), and
//   phase 1  every chunk c >= 1 multiplies its own matrices (L - 1 steps, all chunks side by side): the last chunk's
//            products are final results and are stored as in phase 0; a middle chunk keeps only its total
//            T_c = mats[b_c] ... mats[b_c + L - 1], parked in out[b_c + 1], a slot phase 3 rewrites;
//   phase 2  one chain over the totals (C - 2 steps): out[b_c] = T_c @ out[b_c + L] for c = C-2 ... 1, which are the
//            final suffix products at the chunk boundaries (the kernel runs it with mats = the parked totals);
//   phase 3  every chunk c <= C-2 restarts the chain from out[b_{c+1}] through its own matrices (L - 1 steps, all
//            chunks side by side), storing each product.
// The cotangents, if asked for, are then the finished products applied to g (suffix_apply_kernel).
// About twice the products, a dependent depth of 2L + C - 4 instead of K - 1, no scratch memory, no atomics; the
// summation order is fixed by (K, L), so reruns are bit-identical.
struct ScanPlan {
    int phase;  // 0: whole chain; 1, 2, 3: see above
    int L;      // matrices per chunk (>= 2)
    int C;      // chunks (>= 3)
    // One level of the log-depth form of phase 2 (MODE 3): element c = 1 .. C-2 lives in slot out[b_c + rd], the
    // last element is out[b_{C-1}]; the level writes elem[c] @ elem[c + off] (or elem[c] itself where c + off is
    // past the last element) to out[b_c + wr].
    int off, rd, wr;
    int s;      // chunk boundaries b_c = cL - s (0 or 1)
};

// MODE 0: phase 0 only; every switch below is a compile-time constant, which keeps the whole-chain kernel at its
// register count.  MODE 1: phases 1 and 3 (switches at run time, unit strides).  MODE 2: phase 2 (strided).
// MODE 3: one level of phase 2 in log-depth form (one product per workgroup, all chunks side by side).
template <typename Tin, int D, int RT, int CB, bool COT, int MODE>
__global__ __launch_bounds__(64 * (D / RT)) void scan_mfma_kernel(
    const Tin* __restrict__ mats, float* __restrict__ out, const float* __restrict__ g,
    float* __restrict__ cot, int B, int K, ScanPlan plan) {
    constexpr int NW = D / RT;          // waves per workgroup
    constexpr int NT = 64 * NW;         // threads
    constexpr int RTILES = RT / 32;
    constexpr int CTILES = CB / 32;
    constexpr int NB = D / CB;          // column blocks per batch element
    constexpr int PITCH = D + 4;
    constexpr int NCH = D / 32;         // k chunks per step
    constexpr size_t DD = (size_t)D * D;

    extern __shared__ __align__(16) float lds[];  // [2][CB][PITCH], then (COT) [2][D]
    float* vbuf = lds + 2 * CB * PITCH;

    // A launch covers E = B * (segments per batch element) chains.  With at least 8 of them the workgroups are
    // dealt round-robin to the 8 XCDs so that all column blocks of one chain get ids that are equal mod 8 and
    // share one L2; smaller launches are sized exactly.
    const int nseg = MODE == 1 ? plan.C - 1 : MODE == 3 ? plan.C - 2 : 1;
    const int E = B * nseg;
    const int id = blockIdx.x;
    int e, c0;
    if (E >= 8) {
        const int slot = id >> 3;
        e = (slot / NB) * 8 + (id & 7);
        c0 = (slot % NB) * CB;
    } else {
        e = id / NB;
        c0 = (id % NB) * CB;
    }
    if (e >= E) return;
    const int b = e / nseg;
    const int seg = e - b * nseg;

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int m = lane & 31;
    const int h = lane >> 5;
    const int row0 = wave * RT;

    float* out_b = out + (size_t)b * (K + 1) * DD;
    // The chain of this workgroup: steps r = r_top ... r_lo multiply a_base[r * a_stride] onto the running suffix
    // and store it at o_base[r * o_stride]; the suffix starts as the matrix `init_a` (storage type) or `init_s`
    // (fp32, a product computed earlier).
    const Tin* a_base = mats + (size_t)b * K * DD;
    float* o_base = out_b;
    const Tin* init_a = nullptr;
    const float* init_s = nullptr;
    int r_top, r_lo = 0;
    bool write_tail = false;   // the start matrix and the identity behind it are results (out[K - 1], out[K])
    bool store_all = true;     // every step's product is a result
    // the cotangent chain rides on the whole-chain form only; the chunk phases share no chain to carry it
    static_assert(MODE == 0 || !COT, "chunk phases carry no cotangent chain");
    size_t stride_rt = DD;
    if constexpr (MODE == 0) {
        init_a = a_base + (size_t)(K - 1) * DD;
        r_top = K - 2;
        write_tail = true;
    } else if constexpr (MODE == 1) {
        if (plan.phase == 1) {
            const int c = seg + 1;
            const bool last = c == plan.C - 1;
            const int end = last ? K : (c + 1) * plan.L - plan.s;
            init_a = a_base + (size_t)(end - 1) * DD;
            r_top = end - 2;
            r_lo = c * plan.L - plan.s;
            write_tail = last;
            store_all = last;
        } else {
            const int c = seg;
            init_s = out_b + (size_t)((c + 1) * plan.L - plan.s) * DD;
            r_top = (c + 1) * plan.L - plan.s - 1;
            r_lo = c == 0 ? 0 : c * plan.L - plan.s + 1;   // the chunk's first product is a phase 2 result already
        }
    } else if constexpr (MODE == 3) {
        const int c = seg + 1;
        const float* left = out_b + (size_t)(c * plan.L - plan.s + plan.rd) * DD;
        float* dst = out_b + (size_t)(c * plan.L - plan.s + plan.wr) * DD;
        const int partner = c + plan.off;
        if (partner > plan.C - 1) {
            // nothing to the right at this distance: the element is complete, it moves to the level's output slot
            for (int idx = threadIdx.x; idx < D * CB / 4; idx += NT) {
                const int row = idx / (CB / 4), q = idx % (CB / 4);
                *reinterpret_cast<f32x4*>(dst + (size_t)row * D + c0 + 4 * q) =
                    *reinterpret_cast<const f32x4*>(left + (size_t)row * D + c0 + 4 * q);
            }
            return;
        }
        a_base = reinterpret_cast<const Tin*>(left);
        o_base = dst;
        init_s = partner == plan.C - 1 ? out_b + (size_t)((plan.C - 1) * plan.L - plan.s) * DD
                                       : out_b + (size_t)(partner * plan.L - plan.s + plan.rd) * DD;
        r_top = 0;
    } else {
        // step j multiplies the total parked one slot above the first matrix of chunk j + 1 and stores that first slot
        a_base = reinterpret_cast<const Tin*>(out_b + (size_t)(plan.L - plan.s + 1) * DD);
        o_base = out_b + (size_t)(plan.L - plan.s) * DD;
        stride_rt = (size_t)plan.L * DD;
        init_s = out_b + (size_t)((plan.C - 1) * plan.L - plan.s) * DD;
        r_top = plan.C - 3;
    }
    const bool from_a = MODE == 0 || (MODE == 1 && plan.phase == 1);  // start state: init_a, else init_s
    // distance between the matrices (and the results) of consecutive steps: a constant except in phase 2
    const size_t a_stride = MODE == 2 ? stride_rt : DD;
    const size_t o_stride = a_stride;

    // Start state into St buffer 0 (and, with write_tail, to its place in the result with the identity behind it).
    {
        float* o_last = out_b + (size_t)(K - 1) * DD;
        float* o_eye = out_b + (size_t)K * DD;
        if (MODE != 0) {
            // the chunk phases are short chains: four elements per load, all loads of a thread in flight
            constexpr int Q = CB / 4;
            static_assert((D * Q) % NT == 0, "start-state fill");
#pragma unroll
            for (int u = 0; u < D * Q / NT; ++u) {
                const int idx = tid + u * NT;
                const int row = idx / Q, q = idx % Q;
                const size_t off = (size_t)row * D + c0 + 4 * q;
                const f32x4 v4 = from_a ? load4(init_a + off) : load4(init_s + off);
                if (write_tail) {
                    f32x4 eye = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int t = 0; t < 4; ++t) eye[t] = (row == c0 + 4 * q + t) ? 1.0f : 0.0f;
                    *reinterpret_cast<f32x4*>(o_last + off) = v4;
                    *reinterpret_cast<f32x4*>(o_eye + off) = eye;
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) lds[(4 * q + t) * PITCH + row] = v4[t];
            }
        } else {
        for (int idx = tid; idx < D * CB; idx += NT) {
            const int row = idx / CB;
            const int col = idx % CB;
            const float val = from_a ? to_f32(init_a[row * D + c0 + col]) : init_s[row * D + c0 + col];
            if (write_tail) {
                o_last[row * D + c0 + col] = val;
                o_eye[row * D + c0 + col] = (row == c0 + col) ? 1.0f : 0.0f;
            }
            lds[col * PITCH + row] = val;
        }
        }
        if (COT) {
            // first vector of the chain: (start state) @ g, one row per thread, once per kernel
            const float* g_b = g + (size_t)b * D;
            float* cot_b = cot + (size_t)b * (K + 1) * D;
            for (int row = tid; row < D; row += NT) {
                float acc = 0.0f;
                for (int k4 = 0; k4 < D; k4 += 4) {
                    const f32x4 a4 = from_a ? load4(init_a + row * D + k4) : load4(init_s + row * D + k4);
                    acc = fmaf(a4[0], g_b[k4], acc);
                    acc = fmaf(a4[1], g_b[k4 + 1], acc);
                    acc = fmaf(a4[2], g_b[k4 + 2], acc);
                    acc = fmaf(a4[3], g_b[k4 + 3], acc);
                }
                vbuf[row] = acc;
                if (c0 == 0) {
                    cot_b[(size_t)K * D + row] = g_b[row];
                    cot_b[(size_t)(K - 1) * D + row] = acc;
                }
            }
        }
    }
    __syncthreads();
    if (r_top < r_lo) return;

    // Lane's slice of mats[r]: rows row0 + 32*i + m, k = 32*kc + 16*h + [0, 16).
    auto load_a = [&](f32x4 (&dst)[RTILES][4], const Tin* base) {
#pragma unroll
        for (int i = 0; i < RTILES; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) dst[i][q] = load4(base + (size_t)i * 32 * D + q * 4);
    };
    const Tin* a_lane = a_base + (size_t)(row0 + m) * D + h * 16;  // + r*a_stride + kc*32

    // mats chunks are prefetched RING-1 chunks ahead into a register ring; the ring
    // index of a chunk is kc % RING, the same in every step because RING divides NCH.
    constexpr int RING = (NCH % 4 == 0) ? 4 : 2;
    constexpr int AHEAD = RING - 1;
    f32x4 a_ring[RING][RTILES][4];
    // Chunk number c (0 <= c < AHEAD) counted from the start of step r_top; when NCH == 1
    // chunk 1 is already in the next step.
#pragma unroll
    for (int c = 0; c < AHEAD; ++c) {
        const int rr = r_top - c / NCH;
        load_a(a_ring[c % RING], a_lane + (size_t)(rr > r_lo ? rr : r_lo) * a_stride + (c % NCH) * 32);
    }

    int cur = 0;
    for (int r = r_top; r >= r_lo; r -= (NCH == 1 ? 2 : 1)) {
        // NCH == 1 runs two steps per trip so ring indices stay compile-time constants.
#pragma unroll
        for (int sub = 0; sub < (NCH == 1 ? 2 : 1); ++sub) {
        const int rs = r - sub;
        if (rs < r_lo) break;
        f32x16 acc[RTILES][CTILES];
#pragma unroll
        for (int i = 0; i < RTILES; ++i)
#pragma unroll
            for (int j = 0; j < CTILES; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

        const float* st = lds + cur * (CB * PITCH) + m * PITCH + h * 16;
        const float* v_old = vbuf + cur * D + h * 16;
        float vdot[RTILES];
#pragma unroll
        for (int i = 0; i < RTILES; ++i) vdot[i] = 0.0f;
        const Tin* a_r = a_lane + (size_t)rs * a_stride;
        // Chunks past the end of this step belong to the next step's matrix (a harmless re-read of
        // the last one after the very last step).
        const Tin* a_wrap = a_lane + (size_t)(rs > r_lo ? rs - 1 : r_lo) * a_stride;
#pragma unroll
        for (int kc = 0; kc < NCH; ++kc) {
            const int slot = (NCH == 1 ? sub : kc) % RING;
            const int ahead = kc + AHEAD;
            load_a(a_ring[(slot + AHEAD) % RING], ahead < NCH ? a_r + ahead * 32 : a_wrap + (ahead - NCH) * 32);
            f32x4 bfrag[CTILES][4];
#pragma unroll
            for (int j = 0; j < CTILES; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    bfrag[j][q] = *reinterpret_cast<const f32x4*>(st + j * 32 * PITCH + kc * 32 + q * 4);
            // Blocked summation: the 32 products of this k chunk are summed in a fresh
            // accumulator and added to the running total once, so a total takes D/32
            // roundings at full magnitude per step instead of D/2.
            f32x16 part[RTILES][CTILES];
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int t = 0; t < 4; ++t)
#pragma unroll
                    for (int i = 0; i < RTILES; ++i)
#pragma unroll
                        for (int j = 0; j < CTILES; ++j) {
                            if (q == 0 && t == 0) {
#pragma unroll
                                for (int e = 0; e < 16; ++e) part[i][j][e] = 0.0f;
                            }
                            part[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(
                                a_ring[slot][i][q][t], bfrag[j][q][t], part[i][j], 0, 0, 0);
                        }
#pragma unroll
            for (int i = 0; i < RTILES; ++i)
#pragma unroll
                for (int j = 0; j < CTILES; ++j)
#pragma unroll
                    for (int e = 0; e < 16; ++e) acc[i][j][e] += part[i][j][e];
            if (COT) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x4 v4 = *reinterpret_cast<const f32x4*>(v_old + kc * 32 + q * 4);
#pragma unroll
                    for (int i = 0; i < RTILES; ++i)
#pragma unroll
                        for (int t = 0; t < 4; ++t) vdot[i] = fmaf(a_ring[slot][i][q][t], v4[t], vdot[i]);
                }
            }
            // Keep chunks from being interleaved: it only lengthens register live ranges.
            __builtin_amdgcn_sched_barrier(0);
        }

        // A chunk that only forms its total parks it one slot above its first matrix (phase 1).
        const bool store = store_all || rs == r_lo;
        float* o_r = o_base + (size_t)(store_all ? rs : rs + 1) * o_stride;
        float* st_new = lds + (cur ^ 1) * (CB * PITCH);
#pragma unroll
        for (int i = 0; i < RTILES; ++i)
#pragma unroll
            for (int j = 0; j < CTILES; ++j)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int row = row0 + i * 32 + g * 8 + h * 4;
                    const int col = j * 32 + m;
                    f32x4 v4 = {acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2],
                                acc[i][j][4 * g + 3]};
                    *reinterpret_cast<f32x4*>(st_new + col * PITCH + row) = v4;
                    if (store) {
#pragma unroll
                        for (int t = 0; t < 4; ++t) o_r[(size_t)(row + t) * D + c0 + col] = v4[t];
                    }
                }
        if (COT) {
            float* v_new = vbuf + (cur ^ 1) * D;
            float* cot_r = cot + ((size_t)b * (K + 1) + rs) * D;
#pragma unroll
            for (int i = 0; i < RTILES; ++i) {
                const float total = vdot[i] + __shfl_xor(vdot[i], 32, 64);  // the two k halves of a row
                if (h == 0) {
                    v_new[row0 + i * 32 + m] = total;
                    if (c0 == 0) cot_r[row0 + i * 32 + m] = total;
                }
            }
        }
        // LDS-only barrier: the new block and v are LDS data; a full __syncthreads would also
        // drain the mats prefetch and this step's stores.
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        cur ^= 1;
        }
    }
}

// ---------------------------------------------------------------------------------------
// Generic path: any d (small or not a multiple of 32).  Scalar FMA; the column block
// of the running suffix lives in LDS as S[k][col], double buffered.
// ---------------------------------------------------------------------------------------
template <typename Tin>
__global__ __launch_bounds__(256) void scan_generic_kernel(
    const Tin* __restrict__ mats, float* __restrict__ out, int B, int K, int d, int cb, int nb) {
    extern __shared__ __align__(16) float lds[];  // [2][d][cb]
    const int b = blockIdx.x / nb;
    const int c0 = (blockIdx.x % nb) * cb;
    const int ncol = min(cb, d - c0);
    const int tid = threadIdx.x;
    const Tin* mats_b = mats + (size_t)b * K * d * d;
    float* out_b = out + (size_t)b * (K + 1) * d * d;
    const int nelem = d * ncol;

    {
        const Tin* a_last = mats_b + (size_t)(K - 1) * d * d;
        float* o_last = out_b + (size_t)(K - 1) * d * d;
        float* o_eye = out_b + (size_t)K * d * d;
        for (int idx = tid; idx < nelem; idx += 256) {
            const int row = idx / ncol;
            const int col = idx % ncol;
            const float val = to_f32(a_last[(size_t)row * d + c0 + col]);
            o_last[(size_t)row * d + c0 + col] = val;
            o_eye[(size_t)row * d + c0 + col] = (row == c0 + col) ? 1.0f : 0.0f;
            lds[row * cb + col] = val;
        }
    }
    __syncthreads();

    int cur = 0;
    for (int r = K - 2; r >= 0; --r) {
        const Tin* a = mats_b + (size_t)r * d * d;
        float* o_r = out_b + (size_t)r * d * d;
        const float* s_old = lds + cur * d * cb;
        float* s_new = lds + (cur ^ 1) * d * cb;
        for (int idx = tid; idx < nelem; idx += 256) {
            const int row = idx / ncol;
            const int col = idx % ncol;
            const Tin* a_row = a + (size_t)row * d;
            float acc = 0.0f;
            for (int k = 0; k < d; ++k) acc = fmaf(to_f32(a_row[k]), s_old[k * cb + col], acc);
            s_new[row * cb + col] = acc;
            o_r[(size_t)row * d + c0 + col] = acc;
        }
        __syncthreads();
        cur ^= 1;
    }
}

// K == 0: the result is just the identity.
__global__ void identity_kernel(float* __restrict__ out, int64_t n_mats, int d) {
    const int64_t total = n_mats * d * d;
    for (int64_t idx = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; idx < total;
         idx += (int64_t)gridDim.x * blockDim.x) {
        const int rc = (int)(idx % ((int64_t)d * d));
        out[idx] = (rc / d == rc % d) ? 1.0f : 0.0f;
    }
}

// ---------------------------------------------------------------------------------------
// Cotangent chain: one workgroup per batch element, one mat-vec per step.  A wave
// takes rows wave, wave+NW, ...; lanes run along k so every load instruction reads
// contiguous memory; the 64 partial sums are folded with a butterfly.  The vector
// lives in LDS, double buffered, so a step costs one barrier.  HBM-bound: each
// matrix is read exactly once.
// ---------------------------------------------------------------------------------------
template <typename Tin, bool VEC4>
__global__ __launch_bounds__(512) void cotangent_kernel(
    const Tin* __restrict__ mats, const float* __restrict__ g, float* __restrict__ out, int K, int d) {
    extern __shared__ __align__(16) float lds[];  // [2][dpad]
    const int dpad = (d + 3) & ~3;
    const int b = blockIdx.x;
    const int tid = threadIdx.x;
    const int nw = blockDim.x >> 6;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const Tin* mats_b = mats + (size_t)b * K * d * d;
    float* out_b = out + (size_t)b * (K + 1) * d;

    for (int i = tid; i < d; i += blockDim.x) {
        const float val = g[(size_t)b * d + i];
        lds[i] = val;
        out_b[(size_t)K * d + i] = val;
    }
    __syncthreads();

    int cur = 0;
    for (int r = K - 1; r >= 0; --r) {
        const Tin* a = mats_b + (size_t)r * d * d;
        const float* v_old = lds + cur * dpad;
        float* v_new = lds + (cur ^ 1) * dpad;
        for (int row = wave; row < d; row += nw) {
            const Tin* a_row = a + (size_t)row * d;
            float acc = 0.0f;
            if (VEC4) {
                for (int k = lane * 4; k < d; k += 256) {
                    const f32x4 a4 = load4(a_row + k);
                    const f32x4 v4 = *reinterpret_cast<const f32x4*>(v_old + k);
                    acc = fmaf(a4[0], v4[0], acc);
                    acc = fmaf(a4[1], v4[1], acc);
                    acc = fmaf(a4[2], v4[2], acc);
                    acc = fmaf(a4[3], v4[3], acc);
                }
            } else {
                for (int k = lane; k < d; k += 64) acc = fmaf(to_f32(a_row[k]), v_old[k], acc);
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
            if (lane == 0) {
                v_new[row] = acc;
                out_b[(size_t)r * d + row] = acc;
            }
        }
        __syncthreads();
        cur ^= 1;
    }
}

// ---------------------------------------------------------------------------------------
// Cotangent chain for matrices that fit in LDS in their storage type (rows a multiple of 16 bytes; fp32 up to
// d = 180, 16-bit up to d = 256): a step is bound by the latency of its loads unless they are issued a step ahead.
// The matrix of step r - 1 is fetched into registers while step r is multiplied out of an LDS copy, then
// stored to that copy (two barriers per step, no load on the chain's critical path).  One workgroup of 256
// threads per batch element; a thread multiplies a run of 16-byte pieces of one row, the (at most 32) lanes of a
// row are folded with xor shuffles.
// ---------------------------------------------------------------------------------------
template <typename Tin>
__global__ __launch_bounds__(256) void cotangent_staged_kernel(const Tin* __restrict__ mats, const float* __restrict__ g,
                                                               float* __restrict__ out, int K, int d) {
    constexpr int NT = 256, MAXV = 32;            // 16-byte pieces of a matrix per thread (128 KB / 16 / 256)
    constexpr int EPP = 16 / (int)sizeof(Tin);    // elements per piece: 4 (fp32) or 8 (16-bit)
    typedef unsigned int raw4 __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) char lds_raw[];  // matrix copy [d * d] in Tin, then [2][d] fp32 chain vectors
    Tin* a_lds = reinterpret_cast<Tin*>(lds_raw);
    float* vbuf = reinterpret_cast<float*>(lds_raw + (size_t)d * d * sizeof(Tin));
    const int b = blockIdx.x, tid = threadIdx.x;
    const Tin* mats_b = mats + (size_t)b * K * d * d;
    float* out_b = out + (size_t)b * (K + 1) * d;
    const int pieces = d * d / EPP;
    const int per_row = d / EPP;
    // A row is shared by `parts` adjacent lanes (a power of two, as many as 256 threads allow), each taking a run
    // of `ppp` pieces; lanes start their runs at different pieces so that a wave's 16-byte reads spread over banks.
    int parts = 1;
    while (2 * parts * d <= NT && 2 * parts <= per_row) parts <<= 1;
    const int ppp = (per_row + parts - 1) / parts;
    const int row = tid / parts, part = tid % parts;

    for (int i = tid; i < d; i += NT) {
        const float val = g[(size_t)b * d + i];
        vbuf[i] = val;
        out_b[(size_t)K * d + i] = val;
    }
    raw4 next[MAXV];
    auto fetch = [&](int r) __attribute__((always_inline)) {
        const raw4* a = reinterpret_cast<const raw4*>(mats_b + (size_t)r * d * d);
#pragma unroll
        for (int u = 0; u < MAXV; ++u) {
            const int piece = tid + NT * u;
            if (NT * u >= pieces) break;  // uniform: small matrices leave after one or two rounds
            if (piece < pieces) next[u] = a[piece];
        }
    };
    auto commit = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < MAXV; ++u) {
            const int piece = tid + NT * u;
            if (NT * u >= pieces) break;
            if (piece < pieces) reinterpret_cast<raw4*>(a_lds)[piece] = next[u];
        }
    };
    if (K > 0) {
        fetch(K - 1);
        commit();
    }
    __syncthreads();
    int cur = 0;
    for (int r = K - 1; r >= 0; --r) {
        if (r > 0) fetch(r - 1);
        const float* v_old = vbuf + cur * d;
        float* v_new = vbuf + (cur ^ 1) * d;
        float acc = 0.0f;
        if (row < d) {
            const Tin* a_row = a_lds + row * d;
#pragma unroll 4
            for (int i = 0; i < ppp; ++i) {
                int rot = i + row;
                rot -= (rot / ppp) * ppp;
                const int piece = part * ppp + rot;
                if (piece < per_row) {
#pragma unroll
                    for (int q = 0; q < EPP / 4; ++q) {
                        const f32x4 a4 = load4(a_row + EPP * piece + 4 * q);
                        const f32x4 v4 = *reinterpret_cast<const f32x4*>(v_old + EPP * piece + 4 * q);
                        acc = fmaf(a4[0], v4[0], acc);
                        acc = fmaf(a4[1], v4[1], acc);
                        acc = fmaf(a4[2], v4[2], acc);
                        acc = fmaf(a4[3], v4[3], acc);
                    }
                }
            }
        }
        for (int off = parts >> 1; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
        if (row < d && part == 0) {
            v_new[row] = acc;
            out_b[(size_t)r * d + row] = acc;
        }
        __syncthreads();  // every read of the matrix copy and of v_old is done, v_new is complete
        if (r > 0) commit();
        __syncthreads();
        cur ^= 1;
    }
}

// ---------------------------------------------------------------------------------------
// Cotangent chain for d = 256, fp32: the HBM-bound case that matters.  One workgroup of
// 8 waves per batch element; a wave takes rows wave, wave+8, ... (32 per step), one row
// (1 KiB) per load instruction.  The matrices do not depend on the chain, so a wave keeps its
// 32 rows of the next matrix in flight in registers (248 KiB per workgroup) while the current
// ones are multiplied.  The 32 partial sums of a lane are folded across
// the 64 lanes with a halving butterfly (31 exchanges instead of 32 x 6).
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(512) void cotangent256_kernel(const float* __restrict__ mats,
                                                           const float* __restrict__ g,
                                                           float* __restrict__ out, int K) {
    constexpr int D = 256;
    __shared__ __align__(16) float vbuf[2][D];
    const int b = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: row addresses stay scalar
    const float* mats_b = mats + (size_t)b * K * D * D;
    float* out_b = out + (size_t)b * (K + 1) * D;
    if (tid < D) {
        const float val = g[(size_t)b * D + tid];
        vbuf[0][tid] = val;
        out_b[(size_t)K * D + tid] = val;
    }
    if (K == 0) return;
    // Row wave + 8 * i of matrix r, columns 4 * lane .. 4 * lane + 3.
    auto load_row = [&](int r, int i) {
        return *reinterpret_cast<const f32x4*>(mats_b + (size_t)r * D * D + (size_t)(wave + 8 * i) * D + 4 * lane);
    };
    // LDS writes visible to the workgroup; loads already in flight are NOT waited for
    // (a full __syncthreads would drain them together with the stores of the step).
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    f32x4 buf[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) buf[i] = load_row(K - 1, i);
    lds_barrier();
    int cur = 0;
    for (int r = K - 1; r >= 0; --r) {
        const f32x4 vv = *reinterpret_cast<const f32x4*>(&vbuf[cur][4 * lane]);
        const int r_next = r > 0 ? r - 1 : 0;  // a harmless re-read at the end
        float vals[32];
        // Each register is refilled with the same row of the next matrix as soon as it has been used: 31 of the
        // wave's 32 rows are in flight at any time.
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            vals[i] = fmaf(buf[i][3], vv[3], fmaf(buf[i][2], vv[2], fmaf(buf[i][1], vv[1], buf[i][0] * vv[0])));
            buf[i] = load_row(r_next, i);
            __builtin_amdgcn_sched_barrier(0);  // keep the refill next to the use
        }
        // Halving butterfly: after the stage with mask M a lane keeps the half of its values
        // selected by its bit M; at the end lane l holds row index l >> 1 summed over all lanes.
        auto stage = [&](auto half_tag) {
            constexpr int HALF = decltype(half_tag)::value;  // values kept; also the lane bit of this stage
            const bool up = (lane & (2 * HALF)) != 0;
            float got[HALF];
#pragma unroll
            for (int i = 0; i < HALF; ++i) got[i] = __shfl_xor(up ? vals[i] : vals[i + HALF], 2 * HALF, 64);
#pragma unroll
            for (int i = 0; i < HALF; ++i) vals[i] = (up ? vals[i + HALF] : vals[i]) + got[i];
        };
        stage(std::integral_constant<int, 16>{});
        stage(std::integral_constant<int, 8>{});
        stage(std::integral_constant<int, 4>{});
        stage(std::integral_constant<int, 2>{});
        stage(std::integral_constant<int, 1>{});
        const float total = vals[0] + __shfl_xor(vals[0], 1, 64);
        if ((lane & 1) == 0) {
            const int row = wave + 8 * (lane >> 1);
            vbuf[cur ^ 1][row] = total;
            out_b[(size_t)r * D + row] = total;
        }
        lds_barrier();
        cur ^= 1;
    }
}

// The same chain for 16-bit storage: a row is 512 bytes, so a load instruction covers two rows (lane half = row,
// 8 elements per lane) and a wave's 32 rows are 16 registers in flight; the 16 partial sums of a lane are folded
// across the 32 lanes of its half.
template <typename Tin>
__global__ __launch_bounds__(512) void cotangent256_half_kernel(const Tin* __restrict__ mats,
                                                                const float* __restrict__ g, float* __restrict__ out,
                                                                int K) {
    constexpr int D = 256;
    typedef unsigned int raw4 __attribute__((ext_vector_type(4)));
    __shared__ __align__(16) float vbuf[2][D];
    const int b = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, sub = lane >> 5, piece = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const Tin* mats_b = mats + (size_t)b * K * D * D;
    float* out_b = out + (size_t)b * (K + 1) * D;
    if (tid < D) {
        const float val = g[(size_t)b * D + tid];
        vbuf[0][tid] = val;
        out_b[(size_t)K * D + tid] = val;
    }
    if (K == 0) return;
    // Row wave + 8 * (2 i + sub) of matrix r, elements 8 * piece .. 8 * piece + 7.
    auto load_row = [&](int r, int i) {
        return *reinterpret_cast<const raw4*>(mats_b + (size_t)r * D * D + (size_t)(wave + 8 * (2 * i + sub)) * D + 8 * piece);
    };
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    raw4 buf[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) buf[i] = load_row(K - 1, i);
    lds_barrier();
    int cur = 0;
    for (int r = K - 1; r >= 0; --r) {
        const f32x4 v_lo = *reinterpret_cast<const f32x4*>(&vbuf[cur][8 * piece]);
        const f32x4 v_hi = *reinterpret_cast<const f32x4*>(&vbuf[cur][8 * piece + 4]);
        const int r_next = r > 0 ? r - 1 : 0;  // a harmless re-read at the end
        float vals[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const Tin* e = reinterpret_cast<const Tin*>(&buf[i]);
            float acc = to_f32(e[0]) * v_lo[0];
#pragma unroll
            for (int q = 1; q < 4; ++q) acc = fmaf(to_f32(e[q]), v_lo[q], acc);
#pragma unroll
            for (int q = 0; q < 4; ++q) acc = fmaf(to_f32(e[4 + q]), v_hi[q], acc);
            vals[i] = acc;
            buf[i] = load_row(r_next, i);
            __builtin_amdgcn_sched_barrier(0);  // keep the refill next to the use
        }
        // Halving butterfly inside each 32-lane half: lane `piece` ends with value index piece >> 1.
        auto stage = [&](auto half_tag) {
            constexpr int HALF = decltype(half_tag)::value;
            const bool up = (lane & (2 * HALF)) != 0;
            float got[HALF];
#pragma unroll
            for (int i = 0; i < HALF; ++i) got[i] = __shfl_xor(up ? vals[i] : vals[i + HALF], 2 * HALF, 64);
#pragma unroll
            for (int i = 0; i < HALF; ++i) vals[i] = (up ? vals[i + HALF] : vals[i]) + got[i];
        };
        stage(std::integral_constant<int, 8>{});
        stage(std::integral_constant<int, 4>{});
        stage(std::integral_constant<int, 2>{});
        stage(std::integral_constant<int, 1>{});
        const float total = vals[0] + __shfl_xor(vals[0], 1, 64);
        if ((lane & 1) == 0) {
            const int row = wave + 8 * (2 * (piece >> 1) + sub);
            vbuf[cur ^ 1][row] = total;
            out_b[(size_t)r * D + row] = total;
        }
        lds_barrier();
        cur ^= 1;
    }
}

// ---------------------------------------------------------------------------------------
// The d = 256 chain on FOUR workgroups per batch element, for batches that would otherwise leave three quarters
// of the chip idle (a chain is one workgroup above, and a CU streams only ~50 GB/s on its own).  Workgroup `part`
// of a group owns rows 64 part .. 64 part + 63 of every step's vector: eight streaming waves of eight rows each keep
// their rows of the next matrices in flight (the same bytes in flight per CU as above, four matrices deep for fp32,
// eight for 16-bit storage), and each step's 256-vector is exchanged through the result array itself: the owner
// stores its 64 entries of out[b, r] (which are results anyway), the three partners pick them up from there.  The
// array is filled with a marker word before the launch (a NaN payload no arithmetic produces; a result that
// happened to equal it is stored as the canonical NaN instead), so a reader knows an entry has arrived when the
// word differs from the marker: the data is its own flag, no ordering between two locations is relied on, and no
// scratch memory is needed.  Stores and polls are agent-scope atomics (they bypass the non-coherent cache levels).
//
// The polls are made by a NINTH wave that does nothing else: loads return in order, so a streaming wave that
// waited for a polled word would drain the matrix rows it has in flight on every step.
//
// Termination.  The four workgroups of a group have block ids that are equal mod 8 (one XCD, one L2) and the grid
// is only launched when all of it is resident at once (4 B workgroups <= CUs).  A reader that has polled
// `spin_limit` times without success stops waiting and computes the missing entry itself from the matrix row and
// the vector it already holds, so every wave reaches every barrier whatever the partners do; the result is then
// still correct to rounding (that entry is summed in another order than its owner's).
// ---------------------------------------------------------------------------------------
using scan_col::kChainMarker;
// polls (with a short sleep each) before a reader stops waiting for a partner: of the order of ten milliseconds
constexpr int kChainSpinLimit = 1 << 14;
// LBI_COT_SPIN_LIMIT overrides it (0: a reader never waits and forms every entry itself; for tests of that path)
inline int chain_spin_limit() {
    static const int limit =
        std::getenv("LBI_COT_SPIN_LIMIT") ? std::atoi(std::getenv("LBI_COT_SPIN_LIMIT")) : kChainSpinLimit;
    return limit;
}

__global__ __launch_bounds__(256) void fill_words_kernel(unsigned* __restrict__ p, size_t n, unsigned value) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
        p[i] = value;
}

template <typename Tin>
__global__ __launch_bounds__(576) void cotangent256_group_kernel(const Tin* __restrict__ mats,
                                                                 const float* __restrict__ g, float* __restrict__ out,
                                                                 int B, int K, int spin_limit) {
    constexpr int D = 256, G = 4, ROWS = D / G, RPW = ROWS / 8;  // 64 rows per workgroup, 8 per streaming wave
    constexpr bool WIDE = sizeof(Tin) == 4;
    constexpr int RPL = WIDE ? 1 : 2;    // rows per load instruction (a 16-bit row is 512 bytes: one per lane half)
    constexpr int LPM = RPW / RPL;       // load instructions per wave and matrix: 8 / 4
    constexpr int DEPTH = 32 / LPM;      // matrices in flight: 4 / 8 (32 registers of 16 bytes either way)
    constexpr int EPL = WIDE ? 4 : 8;    // elements per lane and load
    typedef unsigned int raw4 __attribute__((ext_vector_type(4)));
    __shared__ __align__(16) float vbuf[2][D];
    const int id = blockIdx.x;
    const int b = (id >> 5) * 8 + (id & 7);
    const int part = (id >> 3) & 3;
    if (b >= B) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int sub = WIDE ? 0 : lane >> 5, piece = WIDE ? lane : lane & 31;
    const Tin* mats_b = mats + (size_t)b * K * D * D;
    float* out_b = out + (size_t)b * (K + 1) * D;
    const int row0 = part * ROWS;
    if (tid < D) {
        const float val = g[(size_t)b * D + tid];
        vbuf[0][tid] = val;
        if (tid >= row0 && tid < row0 + ROWS) out_b[(size_t)K * D + tid] = val;
    }
    if (K == 0) return;
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    if (wave == 8) {
        // ---- the exchange wave: three foreign entries per lane and step
        int idx[3];
#pragma unroll
        for (int e = 0; e < 3; ++e) {
            const int f = lane + 64 * e;
            idx[e] = f < row0 ? f : f + ROWS;
        }
        lds_barrier();
        int cur = 0;
        for (int r = K - 1; r >= 0; --r) {
            unsigned* row_words = reinterpret_cast<unsigned*>(out_b + (size_t)r * D);
            unsigned got[3] = {kChainMarker, kChainMarker, kChainMarker};
            int spins = 0;
            while (true) {
                bool all = true;
#pragma unroll
                for (int e = 0; e < 3; ++e)
                    if (got[e] == kChainMarker) {
                        got[e] = __hip_atomic_load(row_words + idx[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        all = all && got[e] != kChainMarker;
                    }
                if (all) break;
                if (++spins > spin_limit) {
                    // the partner has not delivered: this entry from the matrix row and the vector at hand
#pragma unroll
                    for (int e = 0; e < 3; ++e)
                        if (got[e] == kChainMarker) {
                            const Tin* a_row = mats_b + (size_t)r * D * D + (size_t)idx[e] * D;
                            float acc = 0.0f;
                            for (int k = 0; k < D; k += 4) {
                                const f32x4 a4 = load4(a_row + k);
                                const f32x4 v4 = *reinterpret_cast<const f32x4*>(&vbuf[cur][k]);
                                acc = fmaf(a4[3], v4[3], fmaf(a4[2], v4[2], fmaf(a4[1], v4[1], fmaf(a4[0], v4[0], acc))));
                            }
                            got[e] = __float_as_uint(acc);
                        }
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
            }
#pragma unroll
            for (int e = 0; e < 3; ++e) vbuf[cur ^ 1][idx[e]] = __uint_as_float(got[e]);
            lds_barrier();
            cur ^= 1;
        }
        return;
    }

    // ---- streaming waves.  Load i of matrix r: row row0 + wave + 8 * (RPL * i + sub), elements EPL * piece ...
    auto load_row = [&](int r, int i) {
        return *reinterpret_cast<const raw4*>(mats_b + (size_t)r * D * D +
                                              (size_t)(row0 + wave + 8 * (RPL * i + sub)) * D + EPL * piece);
    };
    raw4 buf[DEPTH][LPM];
#pragma unroll
    for (int s = 0; s < DEPTH; ++s)
#pragma unroll
        for (int i = 0; i < LPM; ++i) buf[s][i] = load_row(K - 1 - s > 0 ? K - 1 - s : 0, i);
    lds_barrier();
    int cur = 0;
    auto step = [&](auto slot_tag, int r) __attribute__((always_inline)) {
        constexpr int S = decltype(slot_tag)::value;
        const f32x4 v_lo = *reinterpret_cast<const f32x4*>(&vbuf[cur][EPL * piece]);
        f32x4 v_hi = v_lo;
        if (!WIDE) v_hi = *reinterpret_cast<const f32x4*>(&vbuf[cur][EPL * piece + 4]);
        const int r_fill = r - DEPTH > 0 ? r - DEPTH : 0;  // harmless re-reads at the end
        float vals[LPM];
#pragma unroll
        for (int i = 0; i < LPM; ++i) {
            if (WIDE) {
                const raw4 w = buf[S][i];
                vals[i] = fmaf(__uint_as_float(w[3]), v_lo[3],
                               fmaf(__uint_as_float(w[2]), v_lo[2],
                                    fmaf(__uint_as_float(w[1]), v_lo[1], __uint_as_float(w[0]) * v_lo[0])));
            } else {
                const Tin* e = reinterpret_cast<const Tin*>(&buf[S][i]);
                float acc = to_f32(e[0]) * v_lo[0];
#pragma unroll
                for (int q = 1; q < 4; ++q) acc = fmaf(to_f32(e[q]), v_lo[q], acc);
#pragma unroll
                for (int q = 0; q < 4; ++q) acc = fmaf(to_f32(e[4 + q]), v_hi[q], acc);
                vals[i] = acc;
            }
            buf[S][i] = load_row(r_fill, i);
            __builtin_amdgcn_sched_barrier(0);  // keep the refill next to the use
        }
        // halving butterfly over the lane bits 2 * HALF, then plain folds over the lane bits no value index uses
        auto stage = [&](auto half_tag) {
            constexpr int HALF = decltype(half_tag)::value;
            const bool up = (lane & (2 * HALF)) != 0;
            float got[HALF];
#pragma unroll
            for (int i = 0; i < HALF; ++i) got[i] = __shfl_xor(up ? vals[i] : vals[i + HALF], 2 * HALF, 64);
#pragma unroll
            for (int i = 0; i < HALF; ++i) vals[i] = (up ? vals[i + HALF] : vals[i]) + got[i];
        };
        if (WIDE) stage(std::integral_constant<int, 4>{});
        stage(std::integral_constant<int, 2>{});
        stage(std::integral_constant<int, 1>{});
        float total = vals[0] + __shfl_xor(vals[0], 1, 64);
        if (WIDE) {
            total += __shfl_xor(total, 16, 64);
            total += __shfl_xor(total, 32, 64);
        } else {
            total += __shfl_xor(total, 8, 64);
            total += __shfl_xor(total, 16, 64);
        }
        const bool holder = WIDE ? (lane & 0x31) == 0 : (piece & 0x19) == 0;
        if (holder) {
            const int vi = WIDE ? (lane >> 1) & 7 : (piece >> 1) & 3;
            const int row = row0 + wave + 8 * (RPL * vi + sub);
            unsigned bits = __float_as_uint(total);
            if (bits == kChainMarker) bits = 0x7fc00000u;
            vbuf[cur ^ 1][row] = __uint_as_float(bits);
            __hip_atomic_store(reinterpret_cast<unsigned*>(out_b + (size_t)r * D + row), bits, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
        lds_barrier();
        cur ^= 1;
    };
    auto steps = [&](int r_base, auto... slot_tags) __attribute__((always_inline)) {
        // slots 0 .. DEPTH-1 hold matrices r_base, r_base - 1, ...; all waves leave together at the chain's end
        (void)std::initializer_list<int>{(r_base - decltype(slot_tags)::value >= 0
                                              ? (step(slot_tags, r_base - decltype(slot_tags)::value), 0)
                                              : 0)...};
    };
    for (int r_base = K - 1; r_base >= 0; r_base -= DEPTH) {
        if constexpr (DEPTH == 4)
            steps(r_base, std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{},
                  std::integral_constant<int, 2>{}, std::integral_constant<int, 3>{});
        else
            steps(r_base, std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{},
                  std::integral_constant<int, 2>{}, std::integral_constant<int, 3>{},
                  std::integral_constant<int, 4>{}, std::integral_constant<int, 5>{},
                  std::integral_constant<int, 6>{}, std::integral_constant<int, 7>{});
    }
}

// cot[b, r] = out[b, r] @ g[b] for M matrices per batch element: the cotangents of the K-parallel scan, whose
// chunks have no common chain to carry them (M = K + 1; the identity tail gives cot[b, K] = g[b]), and the
// entry point lbi_suffix_apply.  One workgroup per (b, r), or per block of rows of it when there are few matrices
// (launch_suffix_apply); a wave takes four rows at a time, lanes along k (16-byte loads when d is a multiple of 4),
// butterfly fold.
template <bool VEC4>
__global__ __launch_bounds__(256) void suffix_apply_kernel(const float* __restrict__ out, const float* __restrict__ g,
                                                           float* __restrict__ cot, int M, int d, int rows_per_block,
                                                           int parts) {
    const int mat_id = blockIdx.x / parts;
    const int row_begin = (blockIdx.x - mat_id * parts) * rows_per_block;
    const int row_end = row_begin + rows_per_block < d ? row_begin + rows_per_block : d;
    const int b = mat_id / M;
    const float* mat = out + (size_t)mat_id * d * d;
    const float* g_b = g + (size_t)b * d;
    float* cot_r = cot + (size_t)mat_id * d;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // four rows of a wave per trip, so that four loads per lane are in flight; each row's sum runs in the same
    // order whatever the split
    for (int row = row_begin + wave; row < row_end; row += 16) {
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (VEC4) {
            for (int k = lane * 4; k < d; k += 256) {
                const f32x4 v4 = *reinterpret_cast<const f32x4*>(g_b + k);
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    if (row + 4 * u < row_end) {
                        const f32x4 a4 = *reinterpret_cast<const f32x4*>(mat + (size_t)(row + 4 * u) * d + k);
                        acc[u] = fmaf(a4[0], v4[0], acc[u]);
                        acc[u] = fmaf(a4[1], v4[1], acc[u]);
                        acc[u] = fmaf(a4[2], v4[2], acc[u]);
                        acc[u] = fmaf(a4[3], v4[3], acc[u]);
                    }
                }
            }
        } else {
            for (int k = lane; k < d; k += 64) {
                const float v = g_b[k];
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (row + 4 * u < row_end) acc[u] = fmaf(mat[(size_t)(row + 4 * u) * d + k], v, acc[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) acc[u] += __shfl_xor(acc[u], off, 64);
            if (lane == 0 && row + 4 * u < row_end) cot_r[row + 4 * u] = acc[u];
        }
    }
}

int launch_suffix_apply(const void* suffix, const void* g, void* cot, int64_t B, int64_t M, int d, hipStream_t stream) {
    // One workgroup per matrix when there are enough matrices to fill the chip several times over; with few of
    // them (one batch element) a matrix is cut into row blocks of 64, 32 or 16 for as many workgroups.
    int rows_per_block = d;
    const int64_t want = 4 * (int64_t)device_compute_units();
    for (int rpb : {64, 32, 16}) {
        if (B * M * ((d + rows_per_block - 1) / rows_per_block) >= want) break;
        if (rpb < d) rows_per_block = rpb;
    }
    const int parts = (d + rows_per_block - 1) / rows_per_block;
    const dim3 grid((unsigned)(B * M * parts));
    if (d % 4 == 0)
        hipLaunchKernelGGL(suffix_apply_kernel<true>, grid, dim3(256), 0, stream, static_cast<const float*>(suffix),
                           static_cast<const float*>(g), static_cast<float*>(cot), (int)M, d, rows_per_block, parts);
    else
        hipLaunchKernelGGL(suffix_apply_kernel<false>, grid, dim3(256), 0, stream, static_cast<const float*>(suffix),
                           static_cast<const float*>(g), static_cast<float*>(cot), (int)M, d, rows_per_block, parts);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

template <typename Tin, int D, int RT, int CB, bool COT, int MODE = 0>
int launch_mfma_cot(const void* mats, void* out, const void* g, void* cot, int B, int K, hipStream_t stream,
                    ScanPlan plan = ScanPlan{0, 0, 0, 0, 0, 0}) {
    constexpr int NW = D / RT;
    constexpr int NB = D / CB;
    constexpr size_t lds_bytes = ((size_t)2 * CB * (D + 4) + (COT ? 2 * D : 0)) * sizeof(float);
    auto kern = scan_mfma_kernel<Tin, D, RT, CB, COT, MODE>;
    if (int rc = ensure_dynamic_lds<&scan_mfma_kernel<Tin, D, RT, CB, COT, MODE>>(lds_bytes)) return rc;
    // chains in this launch (the kernel derives the same number from the plan)
    const int chains = B * (MODE == 1 ? plan.C - 1 : MODE == 3 ? plan.C - 2 : 1);
    const dim3 grid(chains >= 8 ? ((chains + 7) / 8) * 8 * NB : chains * NB);
    hipLaunchKernelGGL(kern, grid, dim3(64 * NW), lds_bytes, stream, static_cast<const Tin*>(mats),
                       static_cast<float*>(out), static_cast<const float*>(g), static_cast<float*>(cot), B, K, plan);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

template <typename Tin, int D, int RT, int CB>
int launch_mfma(const void* mats, void* out, const void* g, void* cot, int B, int K, hipStream_t stream) {
    return cot ? launch_mfma_cot<Tin, D, RT, CB, true>(mats, out, g, cot, B, K, stream)
               : launch_mfma_cot<Tin, D, RT, CB, false>(mats, out, nullptr, nullptr, B, K, stream);
}

// Whether the products of the chunk totals (phase 2) run in log depth: level l multiplies every element by the one
// 2^l places to its right, all chunks side by side, ceil(log2(C - 1)) launches of one step each, where the chain
// takes C - 2 dependent steps.  The levels need the two slots of a chunk that phase 3 rewrites (L >= 3).
inline int total_levels(int C) {
    int levels = 0;
    while ((1 << levels) < C - 1) ++levels;
    return levels;
}
inline bool totals_in_log_depth(int L, int C) {
    static const bool no_log = std::getenv("LBI_SCAN_TOTALS_CHAIN") && std::atoi(std::getenv("LBI_SCAN_TOTALS_CHAIN"));
    return !no_log && L >= 3 && 2 * total_levels(C) <= C - 2;
}

// Chunking of the K-parallel scan: C chunks of L matrices.  The chunked form does twice the products, which is
// free only while the plain form (B * nb workgroups) leaves at least half of the CUs idle (256 on a whole MI355X;
// the count is asked of the runtime).  The dependent depth is 2L - 2 steps of the chunks plus the products of the
// totals: C - 2 steps as a chain, or ceil(log2(C - 1)) launches of one step, each costing about 1.4 steps (12-13 us
// against 9 us at d = 256).  L is the length with the least such depth among those whose chunks still fit two
// workgroups per CU; where they need more than one per CU a step takes 1.7x as long.  Measured at K = 128, d = 256
// (plain -> chunked, ms per call): B = 1: 2.36 -> 0.17 (L = 4; 0.21 at L = 8), 2: 2.36 -> 0.23, 4: 2.37 -> 0.35,
// 8: 2.04 -> 0.59, 16: 2.05 -> 1.14, 32: 2.07 -> 2.3 (not taken); d = 128: B = 1: 0.070 at L = 4 (0.081 at L = 8),
// 16: 0.35 -> 0.19, 48: 0.43 -> 0.57 (not taken).
// Returns false when the plain chain is at least as good.  LBI_SCAN_CHUNK=0 forces the plain chain, n >= 2 chunks of n.
inline bool plan_chunks(int B, int K, int nb, ScanPlan* plan) {
    static const int forced = std::getenv("LBI_SCAN_CHUNK") ? std::atoi(std::getenv("LBI_SCAN_CHUNK")) : -1;
    if (forced == 0 || K < 12) return false;
    int L = 0;
    if (forced > 0) {
        L = forced < 2 ? 2 : forced;
    } else {
        const int cus = device_compute_units();
        const int groups = B * nb;  // workgroups per chunk
        if (groups > cus / 2) return false;
        const int c_one = cus / groups + 1;      // C - 1 chunks side by side at one workgroup per CU
        const int c_two = 2 * cus / groups + 1;  // at two
        float best = 0.0f;
        for (int cand = 2; (K + cand) / cand >= 4; ++cand) {
            const int C = (K + cand) / cand;  // ceil((K + 1) / cand): boundaries at cL - 1
            if (C > c_two) continue;
            float cost = (float)(2 * cand - 2) +
                         (totals_in_log_depth(cand, C) ? 1.4f * (float)total_levels(C) : (float)(C - 2));
            if (C > c_one) cost *= 1.7f;
            if (L == 0 || cost <= best) {  // ties: the longer chunk (fewer launches)
                best = cost;
                L = cand;
            }
        }
        if (L == 0) return false;
    }
    const int C = (K + L) / L;
    if (C < 4) return false;
    plan->L = L;
    plan->C = C;
    plan->s = 1;
    return true;
}

// The three phases of ScanPlan, one launch each on `stream` (they depend on each other in that order), then the
// cotangents from the finished products.
template <typename Tin, int D, int RT, int CB>
int launch_chunked(const void* mats, void* out, const void* g, void* cot, int B, int K, ScanPlan plan,
                   hipStream_t stream) {
    // Phase 2 in log depth (totals_in_log_depth): the levels alternate between the two slots of a chunk that phase 3
    // rewrites anyway (out[cL + 1], where phase 1 parked the total, and out[cL + 2]: L >= 3) and the last one writes
    // out[cL]; no slot is read and written in the same launch.
    const int levels = total_levels(plan.C);
    const bool log_depth = totals_in_log_depth(plan.L, plan.C);
    for (int phase = 1; phase <= 3; ++phase) {
        plan.phase = phase;
        int rc = LBI_OK;
        if (phase != 2) {
            rc = launch_mfma_cot<Tin, D, RT, CB, false, 1>(mats, out, nullptr, nullptr, B, K, stream, plan);
        } else if (!log_depth) {  // operands and results are fp32 products inside `out`
            rc = launch_mfma_cot<float, D, RT, CB, false, 2>(out, out, nullptr, nullptr, B, K, stream, plan);
        } else {
            plan.rd = 1;
            for (int l = 0; l < levels && !rc; ++l) {
                plan.off = 1 << l;
                plan.wr = l == levels - 1 ? 0 : 3 - plan.rd;
                rc = launch_mfma_cot<float, D, RT, CB, false, 3>(out, out, nullptr, nullptr, B, K, stream, plan);
                plan.rd = plan.wr;
            }
        }
        if (rc) return rc;
    }
    if (cot) return launch_suffix_apply(out, g, cot, B, K + 1, D, stream);
    return LBI_OK;
}

template <typename Tin>
int launch_cotangent(const void* mats, const void* g, void* out, int B, int K, int d, hipStream_t stream);

// batch size from which one workgroup per batch element already fills the chip (two per CU: 512 on a whole MI355X)
inline int wide_block_batch() { return 2 * device_compute_units(); }

// g / cot may be null (matrices only).  With them, the MFMA widths run the fused kernel;
// other widths run the generic scan followed by the cotangent chain kernel.
template <typename Tin>
int launch_scan(const void* mats, void* out, const void* g, void* cot, int B, int K, int d, int flags,
                hipStream_t stream) {
    // Few batch elements: one chain per column block leaves most of the chip idle for K - 1 dependent steps, so
    // the chain is cut into chunks that run side by side (ScanPlan), on narrow column blocks (short steps).
    ScanPlan plan{0, 0, 0, 0, 0, 0};
    switch (d) {
        case 256:
            if (plan_chunks(B, K, 8, &plan)) return launch_chunked<Tin, 256, 32, 32>(mats, out, g, cot, B, K, plan, stream);
            break;
        case 128:
            if (plan_chunks(B, K, 4, &plan)) return launch_chunked<Tin, 128, 32, 32>(mats, out, g, cot, B, K, plan, stream);
            break;
        case 64:
            if (plan_chunks(B, K, 2, &plan)) return launch_chunked<Tin, 64, 32, 32>(mats, out, g, cot, B, K, plan, stream);
            break;
        case 32:
            if (plan_chunks(B, K, 1, &plan)) return launch_chunked<Tin, 32, 32, 32>(mats, out, g, cot, B, K, plan, stream);
            break;
        default: break;
    }
    switch (d) {
        case 256: {
            // bf16 storage runs on the 16-bit matrix pipes: the running suffix enters each product as bf16
            // planes, the bf16 matrix as it is, accumulation in fp32.  Two planes (hi + mid, the default) round
            // that operand to 16 significand bits, 256 times finer than the bf16 rounding of the inputs
            // themselves (error against fp64 <= 2e-4 at K=128 where 2e-2 is asked of 16-bit storage), for two
            // thirds of the products of the exact form; LBI_SCAN_EXACT_SUFFIX in `flags` asks for three planes
            // (hi + mid + lo), which are the fp32 value exactly.
            // Matrices only: the column-owner kernel (a wave keeps its 16 columns of the suffix in registers, no
            // barrier between steps), with chain waves for the cotangents (below).  LBI_SCAN_ROW_OWNER=1 forces
            // the row-owner kernel, whose row dot products carry the chain.
            // fp32 storage would need 3 x 3 planes: measured 4 % faster than the fp32-MFMA kernel and slightly
            // less accurate (the part clocks down under dense bf16 MFMA load), so it is opt-in:
            // LBI_SCAN_SPLIT_FP32=1.
            if constexpr (std::is_same<Tin, bf16_raw>::value) {
                static const bool row_owner = std::getenv("LBI_SCAN_ROW_OWNER") && std::atoi(std::getenv("LBI_SCAN_ROW_OWNER"));
                const int planes = (flags & LBI_SCAN_EXACT_SUFFIX) ? 3 : 2;
                if (!cot && !row_owner && K >= 1) return scan_col::launch(mats, out, B, K, planes, stream);
                // With the chain, while all 4 B workgroups are resident at once: the same column-owner kernel with
                // four more waves per workgroup that carry the chain (the four workgroups of a batch element
                // exchange its vector through `cot`, which is filled with the marker word first).  Larger batches
                // take the row-owner kernel, whose chain needs no exchange.
                if (cot && !row_owner && K >= 1 && 4 * B <= device_compute_units()) {
                    const size_t words = (size_t)B * (K + 1) * 256;
                    hipLaunchKernelGGL(fill_words_kernel, dim3((unsigned)((words + 1023) / 1024)), dim3(256), 0, stream,
                                       static_cast<unsigned*>(cot), words, kChainMarker);
                    return scan_col::launch_with_chain(mats, out, g, cot, B, K, planes, chain_spin_limit(), stream);
                }
                return scan_split::launch<Tin>(mats, out, g, cot, B, K, planes, stream);
            }
            if constexpr (std::is_same<Tin, float>::value) {
                static const bool split_fp32 =
                    std::getenv("LBI_SCAN_SPLIT_FP32") && std::atoi(std::getenv("LBI_SCAN_SPLIT_FP32"));
                if (split_fp32) return scan_split::launch<Tin>(mats, out, g, cot, B, K, 3, stream);
            }
            {
                // Up to 32 batch elements the 64-wide blocks leave half the CUs or more without a workgroup: blocks
                // of 32 columns (twice the workgroups, half the step time).
                static const int narrow = std::getenv("LBI_SCAN_NARROW") ? std::atoi(std::getenv("LBI_SCAN_NARROW")) : -1;
                if (narrow < 0 ? B <= device_compute_units() / 8 : narrow != 0) return launch_mfma<Tin, 256, 32, 32>(mats, out, g, cot, B, K, stream);
            }
            return launch_mfma<Tin, 256, 32, 64>(mats, out, g, cot, B, K, stream);
        }
        // Column blocks of one batch element read the same matrices.  With few batch elements, narrow blocks give
        // the chip enough workgroups, and the blocks of an element run side by side and share the matrices in L2.
        // With many, they drift apart and fetch them again (measured 1.7x / 2.4x the input bytes at d = 64 / 128),
        // so one workgroup then takes all columns.
        case 512: {
            // 16 column blocks of 32 per batch element, 8 waves of 64 rows.  The fused form would spill, so the
            // cotangent chain, if asked for, runs as its own kernel behind the matrices.
            if (int rc = launch_mfma<Tin, 512, 64, 32>(mats, out, nullptr, nullptr, B, K, stream)) return rc;
            return cot ? launch_cotangent<Tin>(mats, g, cot, B, K, d, stream) : LBI_OK;
        }
        case 128:
            if (B >= wide_block_batch()) return launch_mfma<Tin, 128, 32, 128>(mats, out, g, cot, B, K, stream);
            return launch_mfma<Tin, 128, 32, 32>(mats, out, g, cot, B, K, stream);
        case 64:
            if (B >= wide_block_batch()) return launch_mfma<Tin, 64, 32, 64>(mats, out, g, cot, B, K, stream);
            return launch_mfma<Tin, 64, 32, 32>(mats, out, g, cot, B, K, stream);
        case 32: return launch_mfma<Tin, 32, 32, 32>(mats, out, g, cot, B, K, stream);
        default: break;
    }
    if (cot) {
        if (int rc = launch_cotangent<Tin>(mats, g, cot, B, K, d, stream)) return rc;
    }
    // Generic: widest column block (<= 32) whose two LDS copies fit in 64 KiB.
    int cb = d < 32 ? d : 32;
    while (cb > 1 && (size_t)2 * d * cb * sizeof(float) > 64 * 1024) cb >>= 1;
    const size_t lds_bytes = (size_t)2 * d * cb * sizeof(float);
    if (lds_bytes > 64 * 1024) return fail(LBI_ERR_UNSUPPORTED, "suffix scan: d=%d is too large (max 8192)", d);
    const int nb = (d + cb - 1) / cb;
    hipLaunchKernelGGL(scan_generic_kernel<Tin>, dim3((unsigned)B * nb), dim3(256), lds_bytes, stream,
                       static_cast<const Tin*>(mats), static_cast<float*>(out), B, K, d, cb, nb);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

template <typename Tin>
int launch_cotangent(const void* mats, const void* g, void* out, int B, int K, int d, hipStream_t stream) {
    const int dpad = (d + 3) & ~3;
    const size_t lds_bytes = (size_t)2 * dpad * sizeof(float);
    if (lds_bytes > 64 * 1024) return fail(LBI_ERR_UNSUPPORTED, "suffix cotangents: d=%d is too large (max 8192)", d);
    const int threads = d >= 128 ? 512 : (d >= 32 ? 256 : 64);
    if (d == 256 && K >= 2 && 4 * B <= device_compute_units()) {
        // few chains: four workgroups per chain, the vector exchanged through the result array (see the kernel)
        // LBI_COT_GROUP=0 keeps one workgroup per chain
        static const int group = std::getenv("LBI_COT_GROUP") ? std::atoi(std::getenv("LBI_COT_GROUP")) : 1;
        const int spin_limit = chain_spin_limit();
        if (group) {
            const size_t words = (size_t)B * (K + 1) * d;
            hipLaunchKernelGGL(fill_words_kernel, dim3((unsigned)((words + 1023) / 1024 > 1024 ? 1024 : (words + 1023) / 1024)),
                               dim3(256), 0, stream, static_cast<unsigned*>(out), words, kChainMarker);
            hipLaunchKernelGGL(cotangent256_group_kernel<Tin>, dim3((unsigned)((B + 7) / 8) * 32), dim3(576), 0, stream,
                               static_cast<const Tin*>(mats), static_cast<const float*>(g), static_cast<float*>(out), B,
                               K, spin_limit);
            LBI_HIP_CHECK(hipGetLastError());
            return LBI_OK;
        }
    }
    if (d == 256 && std::is_same<Tin, float>::value) {
        hipLaunchKernelGGL(cotangent256_kernel, dim3(B), dim3(512), 0, stream, static_cast<const float*>(mats),
                           static_cast<const float*>(g), static_cast<float*>(out), K);
        LBI_HIP_CHECK(hipGetLastError());
        return LBI_OK;
    }
    if constexpr (sizeof(Tin) == 2) if (d == 256) {
        hipLaunchKernelGGL(cotangent256_half_kernel<Tin>, dim3(B), dim3(512), 0, stream, static_cast<const Tin*>(mats),
                           static_cast<const float*>(g), static_cast<float*>(out), K);
        LBI_HIP_CHECK(hipGetLastError());
        return LBI_OK;
    }
    const size_t matrix_bytes = (size_t)d * d * sizeof(Tin);
    constexpr int per_piece = 16 / (int)sizeof(Tin);  // elements in 16 bytes
    if (d % per_piece == 0 && matrix_bytes <= 128 * 1024 && d / per_piece <= 64) {
        const size_t staged_bytes = matrix_bytes + (size_t)2 * d * sizeof(float);  // <= 130 KB
        auto kern = cotangent_staged_kernel<Tin>;
        if (int rc = ensure_dynamic_lds<&cotangent_staged_kernel<Tin>>(staged_bytes)) return rc;
        hipLaunchKernelGGL(kern, dim3(B), dim3(256), staged_bytes, stream, static_cast<const Tin*>(mats),
                           static_cast<const float*>(g), static_cast<float*>(out), K, d);
        LBI_HIP_CHECK(hipGetLastError());
        return LBI_OK;
    }
    if (d % 4 == 0)
        hipLaunchKernelGGL((cotangent_kernel<Tin, true>), dim3(B), dim3(threads), lds_bytes, stream,
                           static_cast<const Tin*>(mats), static_cast<const float*>(g),
                           static_cast<float*>(out), K, d);
    else
        hipLaunchKernelGGL((cotangent_kernel<Tin, false>), dim3(B), dim3(threads), lds_bytes, stream,
                           static_cast<const Tin*>(mats), static_cast<const float*>(g),
                           static_cast<float*>(out), K, d);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

int check_scan_args(const char* what, const void* mats, const void* out, int64_t B, int64_t K, int64_t d,
                    int in_dtype) {
    if (B < 0 || K < 0 || d < 0) return fail(LBI_ERR_INVALID, "%s: negative size (B=%lld K=%lld d=%lld)", what,
                                              (long long)B, (long long)K, (long long)d);
    if (in_dtype != LBI_F32 && in_dtype != LBI_F16 && in_dtype != LBI_BF16)
        return fail(LBI_ERR_INVALID, "%s: mats must have float, half, or bfloat16 dtype (got %d)", what, in_dtype);
    if (B > (1 << 20) || K > (1 << 24) || d > 8192)
        return fail(LBI_ERR_UNSUPPORTED, "%s: size out of range (B=%lld K=%lld d=%lld)", what, (long long)B,
                    (long long)K, (long long)d);
    if ((double)B * (double)(K + 1) * (double)d * (double)d > 9.0e15)
        return fail(LBI_ERR_UNSUPPORTED, "%s: element count overflows", what);
    if (B > 0 && d > 0) {
        if (!out) return fail(LBI_ERR_INVALID, "%s: out is null", what);
        if (K > 0 && !mats) return fail(LBI_ERR_INVALID, "%s: mats is null", what);
    }
    return LBI_OK;
}

}  // namespace
}  // namespace lbi

namespace lbi {
namespace {

int scan_entry(const char* what, const void* mats, void* out, const void* g, void* cot, int64_t B, int64_t K,
               int64_t d, int in_dtype, int out_dtype, int flags, void* stream_v) {
    clear_error();
    if (flags & ~LBI_SCAN_EXACT_SUFFIX) return fail(LBI_ERR_INVALID, "%s: unknown flag bits 0x%x", what, flags);
    if (int rc = check_scan_args(what, mats, out, B, K, d, in_dtype)) return rc;
    if (out_dtype != LBI_F32) return fail(LBI_ERR_UNSUPPORTED, "%s: out_dtype must be LBI_F32", what);
    if (B == 0 || d == 0) return LBI_OK;
    // widths that are a multiple of four run kernels with 16-byte accesses to every operand
    if (d % 4 == 0 && (reinterpret_cast<uintptr_t>(mats) % 16 || reinterpret_cast<uintptr_t>(out) % 16 ||
                       reinterpret_cast<uintptr_t>(g) % 16 || reinterpret_cast<uintptr_t>(cot) % 16))
        return fail(LBI_ERR_INVALID, "%s: mats, out, g and cot must be 16-byte aligned", what);
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    if (K == 0) {
        const int64_t total = B * d * d;
        const int blocks = (int)((total + 255) / 256 > 4096 ? 4096 : (total + 255) / 256);
        hipLaunchKernelGGL(identity_kernel, dim3(blocks), dim3(256), 0, stream, static_cast<float*>(out), B,
                           (int)d);
        LBI_HIP_CHECK(hipGetLastError());
        // the chain of zero matrices is just g
        if (cot) return launch_cotangent<float>(mats, g, cot, (int)B, 0, (int)d, stream);
        return LBI_OK;
    }
    switch (in_dtype) {
        case LBI_F32: return launch_scan<float>(mats, out, g, cot, (int)B, (int)K, (int)d, flags, stream);
        case LBI_F16: return launch_scan<_Float16>(mats, out, g, cot, (int)B, (int)K, (int)d, flags, stream);
        default: return launch_scan<bf16_raw>(mats, out, g, cot, (int)B, (int)K, (int)d, flags, stream);
    }
}

}  // namespace
}  // namespace lbi

extern "C" int lbi_suffix_scan(const void* mats, void* out, int64_t B, int64_t K, int64_t d, int in_dtype,
                               int out_dtype, void* stream_v) {
    return lbi::scan_entry("lbi_suffix_scan", mats, out, nullptr, nullptr, B, K, d, in_dtype, out_dtype, 0, stream_v);
}

extern "C" int lbi_suffix_scan_ex(const void* mats, const void* g, void* out, void* cot, int64_t B, int64_t K,
                                  int64_t d, int in_dtype, int out_dtype, int flags, void* stream_v) {
    using namespace lbi;
    if (B > 0 && d > 0 && ((g == nullptr) != (cot == nullptr))) {
        clear_error();
        return fail(LBI_ERR_INVALID, "lbi_suffix_scan_ex: g and cot must both be given or both be null");
    }
    return scan_entry("lbi_suffix_scan_ex", mats, out, g, cot, B, K, d, in_dtype, out_dtype, flags, stream_v);
}

extern "C" int lbi_suffix_scan_with_cotangents(const void* mats, const void* g, void* out, void* cot, int64_t B,
                                               int64_t K, int64_t d, int in_dtype, int out_dtype, void* stream_v) {
    using namespace lbi;
    if (B > 0 && d > 0 && (!g || !cot)) {
        clear_error();
        return fail(LBI_ERR_INVALID, "lbi_suffix_scan_with_cotangents: g or cot is null");
    }
    return scan_entry("lbi_suffix_scan_with_cotangents", mats, out, g, cot, B, K, d, in_dtype, out_dtype, 0, stream_v);
}

extern "C" int lbi_suffix_cotangents(const void* mats, const void* g, void* out, int64_t B, int64_t K, int64_t d,
                                     int in_dtype, void* stream_v) {
    using namespace lbi;
    clear_error();
    if (int rc = check_scan_args("lbi_suffix_cotangents", mats, out, B, K, d, in_dtype)) return rc;
    if (B == 0 || d == 0) return LBI_OK;
    if (!g) return fail(LBI_ERR_INVALID, "lbi_suffix_cotangents: g is null");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    switch (in_dtype) {
        case LBI_F32: return launch_cotangent<float>(mats, g, out, (int)B, (int)K, (int)d, stream);
        case LBI_F16: return launch_cotangent<_Float16>(mats, g, out, (int)B, (int)K, (int)d, stream);
        default: return launch_cotangent<bf16_raw>(mats, g, out, (int)B, (int)K, (int)d, stream);
    }
}

extern "C" int lbi_suffix_apply(const void* suffix, const void* g, void* out, int64_t B, int64_t M, int64_t d,
                                void* stream_v) {
    using namespace lbi;
    clear_error();
    if (B < 0 || M < 0 || d < 0)
        return fail(LBI_ERR_INVALID, "lbi_suffix_apply: negative size (B=%lld M=%lld d=%lld)", (long long)B,
                    (long long)M, (long long)d);
    if (d > 8192 || (double)B * (double)M > 2.0e9)
        return fail(LBI_ERR_UNSUPPORTED, "lbi_suffix_apply: size out of range (B=%lld M=%lld d=%lld)", (long long)B,
                    (long long)M, (long long)d);
    if (B == 0 || M == 0 || d == 0) return LBI_OK;
    if (!suffix || !g || !out) return fail(LBI_ERR_INVALID, "lbi_suffix_apply: null pointer");
    if (d % 4 == 0 && (reinterpret_cast<uintptr_t>(suffix) % 16 || reinterpret_cast<uintptr_t>(g) % 16))
        return fail(LBI_ERR_INVALID, "lbi_suffix_apply: suffix and g must be 16-byte aligned");
    return launch_suffix_apply(suffix, g, out, B, M, (int)d, static_cast<hipStream_t>(stream_v));
}
