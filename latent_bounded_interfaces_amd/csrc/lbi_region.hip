// Region-level input pullback of a Transformer block: the memory-bound pieces between the
// matrix products (which the host issues as library GEMMs) and the attention pullback.
//
// A cotangent basis carries P directions, so every tensor here is [B, P, T, *] while the
// forward activations it is combined with are [B, T, *]: each kernel reads the activation
// row of (b, t) for all P directions of that token and never materialises a broadcast copy.
// All arithmetic is fp32; 16-bit storage is rounded to nearest-even on the way out.
//
//   rmsnorm_pullback      g_x = r (w o g_y) - x r^3 mean(x o w o g_y)  (+ residual cotangent)
//   gated_mlp_pullback    (up, gate) cotangents of  up * silu(gate)
//   heads_split           [B,P,T,H,Dh] -> [B,P,H,T,Dh]
//   qkv_pullback          dq, dk, dv [B,P,H,T,Dh] -> cotangent of the packed projection
//                         [B,P,T,(H+2Hkv) Dh]: sum over the query heads of a KV group,
//                         transposed rotary embedding, head merge
//   causal_conv1d_pullback  transpose of the depthwise causal convolution over T
#include <hip/hip_runtime.h>

#include "lbi_common.h"

namespace lbi {
namespace region {

template <typename T> __device__ __forceinline__ T from_f32(float x);
template <> __device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <> __device__ __forceinline__ _Float16 from_f32<_Float16>(float x) { return (_Float16)x; }
template <> __device__ __forceinline__ bf16_raw from_f32<bf16_raw>(float x) { return bf16_raw{f32_to_bf16_bits(x)}; }

// x rounded to storage type T and widened again (the value a T-typed tensor would hold).
template <typename T> __device__ __forceinline__ float round_via(float x) { return to_f32(from_f32<T>(x)); }

template <typename T, int VEC> struct Pack;
template <typename T> struct Pack<T, 1> {
    float v[1];
    __device__ __forceinline__ void load(const T* p) { v[0] = to_f32(p[0]); }
    __device__ __forceinline__ void store(T* p) const { p[0] = from_f32<T>(v[0]); }
};
template <typename T> struct Pack<T, 4> {
    float v[4];
    __device__ __forceinline__ void load(const T* p) {
        const f32x4 t = load4(p);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = t[i];
    }
    __device__ __forceinline__ void store(T* p) const;
};
template <> __device__ __forceinline__ void Pack<float, 4>::store(float* p) const {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
}
template <> __device__ __forceinline__ void Pack<_Float16, 4>::store(_Float16* p) const {
    *reinterpret_cast<f16x4*>(p) = f16x4{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
}
template <> __device__ __forceinline__ void Pack<bf16_raw, 4>::store(bf16_raw* p) const {
    *reinterpret_cast<u16x4*>(p) =
        u16x4{f32_to_bf16_bits(v[0]), f32_to_bf16_bits(v[1]), f32_to_bf16_bits(v[2]), f32_to_bf16_bits(v[3])};
}

// Eight 16-bit elements: one 16-byte access.
template <> struct Pack<_Float16, 8> {
    float v[8];
    __device__ __forceinline__ void load(const _Float16* p) {
        const f16x8 h = *reinterpret_cast<const f16x8*>(p);
        v[0] = (float)h[0]; v[1] = (float)h[1]; v[2] = (float)h[2]; v[3] = (float)h[3];
        v[4] = (float)h[4]; v[5] = (float)h[5]; v[6] = (float)h[6]; v[7] = (float)h[7];
    }
    __device__ __forceinline__ void store(_Float16* p) const {
        *reinterpret_cast<f16x8*>(p) = f16x8{(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3],
                                             (_Float16)v[4], (_Float16)v[5], (_Float16)v[6], (_Float16)v[7]};
    }
};
template <> struct Pack<bf16_raw, 8> {
    float v[8];
    __device__ __forceinline__ void load(const bf16_raw* p) {
        const f32x4 w = *reinterpret_cast<const f32x4*>(p);  // four words, two elements each
        v[0] = __uint_as_float(__float_as_uint(w[0]) << 16); v[1] = __uint_as_float(__float_as_uint(w[0]) & 0xffff0000u);
        v[2] = __uint_as_float(__float_as_uint(w[1]) << 16); v[3] = __uint_as_float(__float_as_uint(w[1]) & 0xffff0000u);
        v[4] = __uint_as_float(__float_as_uint(w[2]) << 16); v[5] = __uint_as_float(__float_as_uint(w[2]) & 0xffff0000u);
        v[6] = __uint_as_float(__float_as_uint(w[3]) << 16); v[7] = __uint_as_float(__float_as_uint(w[3]) & 0xffff0000u);
    }
    __device__ __forceinline__ void store(bf16_raw* p) const {
        *reinterpret_cast<u16x8*>(p) =
            u16x8{f32_to_bf16_bits(v[0]), f32_to_bf16_bits(v[1]), f32_to_bf16_bits(v[2]), f32_to_bf16_bits(v[3]),
                  f32_to_bf16_bits(v[4]), f32_to_bf16_bits(v[5]), f32_to_bf16_bits(v[6]), f32_to_bf16_bits(v[7])};
    }
};

// Elements of T in a 16-byte access.
template <typename T> constexpr int wide() { return 16 / (int)sizeof(T); }

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}

// ---------------------------------------------------------------------------------------
// RMSNorm pullback.  One wave per cotangent row (b, p, t); the row is read twice (sums,
// then outputs), the second time from cache.  x is first rounded to the storage type the
// norm ran in (TB), as the forward does.
// ---------------------------------------------------------------------------------------
template <typename TB, typename TX, int VEC>
__global__ __launch_bounds__(256) void rmsnorm_pullback_kernel(const TB* __restrict__ g_out, const TX* __restrict__ x,
                                                               const TB* __restrict__ weight,
                                                               const float* g_residual, float* g_sum,
                                                               TB* __restrict__ g_sum_branch, long long n_rows,
                                                               int P, int T_len, int D, float eps, int res_bcast) {
    const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int lane = threadIdx.x & 63;
    const long long bp = row / T_len;
    const int t = (int)(row - bp * T_len);
    const long long b = bp / P;
    const TB* g_row = g_out + row * D;
    const TX* x_row = x + (b * T_len + t) * D;

    float ss = 0.0f, dot = 0.0f;
    for (int j = lane * VEC; j < D; j += 64 * VEC) {
        Pack<TB, VEC> g, w;
        Pack<TX, VEC> xv;
        g.load(g_row + j);
        w.load(weight + j);
        xv.load(x_row + j);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const float xr = round_via<TB>(xv.v[i]);
            ss = fmaf(xr, xr, ss);
            dot = fmaf(xr, w.v[i] * g.v[i], dot);
        }
    }
    ss = wave_sum(ss);
    dot = wave_sum(dot);
    const float r = rsqrtf(ss / (float)D + eps);
    const float c = r * r * r * dot / (float)D;
    for (int j = lane * VEC; j < D; j += 64 * VEC) {
        Pack<TB, VEC> g, w, ob;
        Pack<TX, VEC> xv;
        Pack<float, VEC> res, of;
        g.load(g_row + j);
        w.load(weight + j);
        xv.load(x_row + j);
        if (g_residual != nullptr) res.load(g_residual + (res_bcast ? bp : row) * D + j);  // [B,P,D] or [B,P,T,D]
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const float xr = round_via<TB>(xv.v[i]);
            float o = r * (w.v[i] * g.v[i]) - xr * c;
            if (g_residual != nullptr) o += res.v[i];
            of.v[i] = o;
            ob.v[i] = o;
        }
        if (g_sum != nullptr) of.store(g_sum + row * D + j);
        if (g_sum_branch != nullptr) ob.store(g_sum_branch + row * D + j);
    }
}

// ---------------------------------------------------------------------------------------
// Gated MLP pullback.  fc1_output rows are [up | gate]; the forward computed
// down_input = up * silu(gate) with silu(gate) rounded to the storage type.
// ---------------------------------------------------------------------------------------
// One workgroup per token (b, t): the activation row is read and its silu terms are formed once,
// then applied to the P cotangent rows of that token.
template <typename T, int VEC>
__global__ __launch_bounds__(256) void gated_mlp_pullback_kernel(const T* __restrict__ g_down_input,
                                                                 const T* __restrict__ fc1_output,
                                                                 T* __restrict__ g_fc1_output, int P, int T_len,
                                                                 int hidden, int g_bcast) {
    const int b = blockIdx.x / T_len, t = blockIdx.x - b * T_len;
    const T* act_row = fc1_output + (long long)blockIdx.x * 2 * hidden;
    const long long row0 = (long long)b * P * T_len + t;  // cotangent row of direction 0
    for (int j = threadIdx.x * VEC; j < hidden; j += blockDim.x * VEC) {
        Pack<T, VEC> up, gate;
        up.load(act_row + j);
        gate.load(act_row + hidden + j);
        float act[VEC], dact[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            const float z = gate.v[i];
            const float sig = 1.0f / (1.0f + __expf(-z));
            act[i] = round_via<T>(z * sig);
            dact[i] = sig * (1.0f + z * (1.0f - sig));
        }
#pragma unroll 4
        for (int p = 0; p < P; ++p) {
            const long long row = row0 + (long long)p * T_len;
            Pack<T, VEC> g, o_up, o_gate;
            g.load(g_down_input + (g_bcast ? (long long)b * P + p : row) * hidden + j);  // [B,P,hidden] or [B,P,T,hidden]
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                o_up.v[i] = g.v[i] * act[i];
                o_gate.v[i] = round_via<T>(g.v[i] * up.v[i]) * dact[i];
            }
            o_up.store(g_fc1_output + row * 2 * hidden + j);
            o_gate.store(g_fc1_output + row * 2 * hidden + hidden + j);
        }
    }
}

// ---------------------------------------------------------------------------------------
// Head split: in [N, T, H, Dh] -> out [N, H, T, Dh]  (N = B * P), 16-byte chunks when Dh allows.
// ---------------------------------------------------------------------------------------
template <typename CHUNK>
__global__ __launch_bounds__(256) void heads_split_kernel(const CHUNK* __restrict__ in, CHUNK* __restrict__ out,
                                                          long long n_chunks, int T_len, int H, int chunks_per_head) {
    const long long o = (long long)blockIdx.x * 256 + threadIdx.x;
    if (o >= n_chunks) return;
    const int c = (int)(o % chunks_per_head);
    long long rest = o / chunks_per_head;
    const int t = (int)(rest % T_len);
    rest /= T_len;
    const int h = (int)(rest % H);
    const long long n = rest / H;
    out[o] = in[((n * T_len + t) * H + h) * chunks_per_head + c];
}

// ---------------------------------------------------------------------------------------
// Packed-projection cotangent from the attention pullback outputs.
//   out[n, t, :] = [ R^T dq[n, 0..H) | R^T sum_group dk | sum_group dv ],  n = (b, p)
// R is the rotary embedding of position t: (e, o) -> (e cos - o sin, e sin + o cos), pairs
// (j, j + Dh/2) or, interleaved, (2j, 2j + 1); R^T: (ge cos + go sin, -ge sin + go cos).
// One thread handles VEC pairs of one rotary head, or 2 VEC value elements.
// ---------------------------------------------------------------------------------------
// Cotangent of the packed projection for one (n, t), one packed head and VEC rotary pairs starting at pair j
// (or 2 VEC value elements): sums the query heads of a key/value group, applies the transposed rotation.
// y0 / y1 are the values at in-head offsets off0.. / off1.. (see qkv_unit_offsets).
template <int VEC, bool INTERLEAVED>
__device__ __forceinline__ void qkv_unit_offsets(bool rotary, int half, int j, int& off0, int& off1) {
    off0 = (rotary && !INTERLEAVED) ? j : 2 * j;
    off1 = (rotary && !INTERLEAVED) ? half + j : 2 * j + VEC;
}

template <typename T, int VEC, bool INTERLEAVED>
__device__ __forceinline__ void qkv_unit_values(const T* __restrict__ dq, const T* __restrict__ dk,
                                                const T* __restrict__ dv, const float* __restrict__ cos_t,
                                                const float* __restrict__ sin_t, long long n, int t, int T_len, int H,
                                                int Hkv, int Dh, int head, int j, float (&y0)[VEC], float (&y1)[VEC]) {
    const int half = Dh / 2;
    const int rep = H / Hkv;
    const bool rotary = head < H + Hkv;
    int off0, off1;
    qkv_unit_offsets<VEC, INTERLEAVED>(rotary, half, j, off0, off1);
    const T* src;
    int first_head, count;
    if (head < H) {
        src = dq; first_head = head; count = 1;
    } else if (head < H + Hkv) {
        src = dk; first_head = (head - H) * rep; count = rep;
    } else {
        src = dv; first_head = (head - H - Hkv) * rep; count = rep;
    }
    float a0[VEC], a1[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) a0[i] = a1[i] = 0.0f;
    for (int g = 0; g < count; ++g) {
        const T* p = src + (((n * H + first_head + g) * T_len) + t) * (long long)Dh;
        Pack<T, VEC> x0, x1;
        x0.load(p + off0);
        x1.load(p + off1);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            a0[i] += x0.v[i];
            a1[i] += x1.v[i];
        }
    }
    if (!rotary) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            y0[i] = a0[i];
            y1[i] = a1[i];
        }
        return;
    }
    Pack<float, VEC> cs, sn;
    cs.load(cos_t + (long long)t * half + j);
    sn.load(sin_t + (long long)t * half + j);
    float ge[VEC], go[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        if (INTERLEAVED) {  // a0|a1 holds pairs (2i, 2i+1) of the 2 VEC span
            const int e = 2 * i, o = 2 * i + 1;
            ge[i] = e < VEC ? a0[e % VEC] : a1[e % VEC];
            go[i] = o < VEC ? a0[o % VEC] : a1[o % VEC];
        } else {
            ge[i] = a0[i];
            go[i] = a1[i];
        }
    }
    float re[VEC], ro[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        // explicit fused steps: every caller rounds the same way whatever the compiler would contract
        re[i] = fmaf(ge[i], cs.v[i], go[i] * sn.v[i]);
        ro[i] = fmaf(go[i], cs.v[i], -(ge[i] * sn.v[i]));
    }
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        if (INTERLEAVED) {
            const int e = 2 * i, o = 2 * i + 1;
            if (e < VEC) y0[e % VEC] = re[i]; else y1[e % VEC] = re[i];
            if (o < VEC) y0[o % VEC] = ro[i]; else y1[o % VEC] = ro[i];
        } else {
            y0[i] = re[i];
            y1[i] = ro[i];
        }
    }
}

template <typename T, int VEC, bool INTERLEAVED>
__global__ __launch_bounds__(256) void qkv_pullback_kernel(const T* __restrict__ dq, const T* __restrict__ dk,
                                                           const T* __restrict__ dv, const float* __restrict__ cos_t,
                                                           const float* __restrict__ sin_t, T* __restrict__ out,
                                                           long long n_units, int T_len, int H, int Hkv, int Dh) {
    const long long unit = (long long)blockIdx.x * 256 + threadIdx.x;
    if (unit >= n_units) return;
    const int half = Dh / 2;
    const int upr = half / VEC;                  // units per head (rotary pair groups, or 2 VEC value elements)
    const int per_token = (H + 2 * Hkv) * upr;
    const long long row = unit / per_token;      // (n, t)
    const int u = (int)(unit - row * per_token);
    const int head = u / upr;                    // packed head index: q heads, then k heads, then v heads
    const int j = (u - head * upr) * VEC;
    const long long n = row / T_len;
    const int t = (int)(row - n * T_len);
    T* o_row = out + row * (long long)(H + 2 * Hkv) * Dh + (long long)head * Dh;
    int off0, off1;
    qkv_unit_offsets<VEC, INTERLEAVED>(head < H + Hkv, half, j, off0, off1);
    float v0[VEC], v1[VEC];
    qkv_unit_values<T, VEC, INTERLEAVED>(dq, dk, dv, cos_t, sin_t, n, t, T_len, H, Hkv, Dh, head, j, v0, v1);
    Pack<T, VEC> y0, y1;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
        y0.v[i] = v0[i];
        y1.v[i] = v1[i];
    }
    y0.store(o_row + off0);
    y1.store(o_row + off1);
}

// The same projection cotangent pulled back through the depthwise causal convolution that follows the packed
// projection (see the transposed convolution below), without storing the intermediate: one thread forms the
// projection cotangent of its 2 VEC channels at RUN + KMAX - 1 consecutive positions and accumulates RUN outputs.
template <typename T, int VEC, int KMAX, int RUN, bool INTERLEAVED, bool EXACT>
__global__ __launch_bounds__(256) void qkv_conv_pullback_kernel(const T* __restrict__ dq, const T* __restrict__ dk,
                                                                const T* __restrict__ dv,
                                                                const float* __restrict__ cos_t,
                                                                const float* __restrict__ sin_t,
                                                                const T* __restrict__ weight, T* __restrict__ out,
                                                                long long n_units, int T_len, int H, int Hkv, int Dh,
                                                                int ksize) {
    const long long unit = (long long)blockIdx.x * 256 + threadIdx.x;
    if (unit >= n_units) return;
    const int half = Dh / 2;
    const int upr = half / VEC;
    const int per_token = (H + 2 * Hkv) * upr;
    const int n_runs = (T_len + RUN - 1) / RUN;
    const int u = (int)(unit % per_token);
    const long long rest = unit / per_token;
    const int s0 = (int)(rest % n_runs) * RUN;
    const long long n = rest / n_runs;
    const int head = u / upr;
    const int j = (u - head * upr) * VEC;
    const int C = (H + 2 * Hkv) * Dh;
    int off0, off1;
    qkv_unit_offsets<VEC, INTERLEAVED>(head < H + Hkv, half, j, off0, off1);
    const int c0 = head * Dh + off0, c1 = head * Dh + off1;

    float tap0[KMAX][VEC], tap1[KMAX][VEC];  // tap[i][e] multiplies the projection cotangent at offset +i
    if (EXACT) {
        // ksize == KMAX: the VEC x KMAX weights of a channel group are one contiguous, aligned span
        Pack<T, VEC> w0[KMAX], w1[KMAX];
#pragma unroll
        for (int u2 = 0; u2 < KMAX; ++u2) {
            w0[u2].load(weight + (long long)c0 * KMAX + u2 * VEC);
            w1[u2].load(weight + (long long)c1 * KMAX + u2 * VEC);
        }
#pragma unroll
        for (int i = 0; i < KMAX; ++i)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int flat = e * KMAX + (KMAX - 1 - i);
                tap0[i][e] = w0[flat / VEC].v[flat % VEC];
                tap1[i][e] = w1[flat / VEC].v[flat % VEC];
            }
    } else {
#pragma unroll
        for (int i = 0; i < KMAX; ++i)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                tap0[i][e] = i < ksize ? to_f32(weight[(long long)(c0 + e) * ksize + (ksize - 1 - i)]) : 0.0f;
                tap1[i][e] = i < ksize ? to_f32(weight[(long long)(c1 + e) * ksize + (ksize - 1 - i)]) : 0.0f;
            }
    }
    float acc0[RUN][VEC], acc1[RUN][VEC];
#pragma unroll
    for (int r = 0; r < RUN; ++r)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc0[r][e] = acc1[r][e] = 0.0f;
    T* o = out + (n * T_len + s0) * (long long)C;
#pragma unroll
    for (int jj = 0; jj < RUN + KMAX - 1; ++jj) {
        float g0[VEC], g1[VEC];
        if (s0 + jj < T_len && jj < RUN + ksize - 1) {
            qkv_unit_values<T, VEC, INTERLEAVED>(dq, dk, dv, cos_t, sin_t, n, s0 + jj, T_len, H, Hkv, Dh, head, j, g0,
                                                 g1);
#pragma unroll
            for (int e = 0; e < VEC; ++e) {  // the stored intermediate of the two-kernel form is rounded to T
                g0[e] = round_via<T>(g0[e]);
                g1[e] = round_via<T>(g1[e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) g0[e] = g1[e] = 0.0f;
        }
#pragma unroll
        for (int r = 0; r < RUN; ++r) {
            const int i = jj - r;
            if (i >= 0 && i < KMAX) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    acc0[r][e] = fmaf(tap0[i][e], g0[e], acc0[r][e]);
                    acc1[r][e] = fmaf(tap1[i][e], g1[e], acc1[r][e]);
                }
            }
        }
        // output jj - (KMAX - 1) has now seen its last row: store it, so only KMAX outputs are live at a time
        const int r = jj - (KMAX - 1);
        if (r >= 0 && r < RUN && s0 + r < T_len) {
            Pack<T, VEC> y0, y1;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                y0.v[e] = acc0[r][e];
                y1.v[e] = acc1[r][e];
            }
            y0.store(o + (long long)r * C + c0);
            y1.store(o + (long long)r * C + c1);
        }
    }
}

// ---------------------------------------------------------------------------------------
// Depthwise causal convolution over T, transposed.
//   forward  y[n, t, c] = sum_j w[c, j] x[n, t + j - (k-1), c]      (x = 0 before the sequence)
//   pullback g_x[n, s, c] = sum_i w[c, k-1-i] g_y[n, s + i, c],  s + i < T
// ---------------------------------------------------------------------------------------
// One thread: VEC channels x RUN consecutive positions, KMAX >= ksize taps held in registers
// (taps past ksize are zero), input rows read once per RUN outputs.
template <typename T, int VEC, int KMAX, int RUN, bool EXACT>
__global__ __launch_bounds__(256) void causal_conv1d_pullback_kernel(const T* __restrict__ g_out,
                                                                     const T* __restrict__ weight, T* __restrict__ g_in,
                                                                     long long n_units, int T_len, int C, int ksize) {
    const long long unit = (long long)blockIdx.x * 256 + threadIdx.x;
    if (unit >= n_units) return;
    const int per_row = C / VEC;
    const int n_runs = (T_len + RUN - 1) / RUN;
    const int c0 = (int)(unit % per_row) * VEC;
    const long long rest = unit / per_row;
    const int s0 = (int)(rest % n_runs) * RUN;
    const long long n = rest / n_runs;

    float tap[KMAX][VEC];  // tap[i][e] multiplies g_out at offset +i
    if (EXACT) {
        // ksize == KMAX: the VEC x KMAX weights of these channels are one contiguous, aligned span
        Pack<T, VEC> wv[KMAX];
#pragma unroll
        for (int u = 0; u < KMAX; ++u) wv[u].load(weight + (long long)c0 * KMAX + u * VEC);
#pragma unroll
        for (int i = 0; i < KMAX; ++i)
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int flat = e * KMAX + (KMAX - 1 - i);
                tap[i][e] = wv[flat / VEC].v[flat % VEC];
            }
    } else {
#pragma unroll
        for (int i = 0; i < KMAX; ++i)
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                tap[i][e] = i < ksize ? to_f32(weight[(long long)(c0 + e) * ksize + (ksize - 1 - i)]) : 0.0f;
    }
    float acc[RUN][VEC];
#pragma unroll
    for (int r = 0; r < RUN; ++r)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[r][e] = 0.0f;
    const long long base = (n * T_len + s0) * C + c0;
#pragma unroll
    for (int j = 0; j < RUN + KMAX - 1; ++j) {
        Pack<T, VEC> g;
        if (s0 + j < T_len && j < RUN + ksize - 1) {
            g.load(g_out + base + (long long)j * C);
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) g.v[e] = 0.0f;
        }
#pragma unroll
        for (int r = 0; r < RUN; ++r) {
            const int i = j - r;
            if (i >= 0 && i < KMAX) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[r][e] = fmaf(tap[i][e], g.v[e], acc[r][e]);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < RUN; ++r) {
        if (s0 + r < T_len) {
            Pack<T, VEC> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o.v[e] = acc[r][e];
            o.store(g_in + base + (long long)r * C);
        }
    }
}

inline unsigned blocks_for(long long units, int per_block) { return (unsigned)((units + per_block - 1) / per_block); }

inline bool fits_grid(long long units, int per_block) {
    return units > 0 && (units + per_block - 1) / per_block <= 0x7fffffffLL;
}

template <typename TB, typename TX>
int launch_rmsnorm(const void* g_out, const void* x, const void* weight, const void* g_residual, void* g_sum,
                   void* g_sum_branch, long long n_rows, int P, int T_len, int D, float eps, int res_bcast,
                   hipStream_t stream) {
    const dim3 grid(blocks_for(n_rows, 4)), block(256);
    if (D % 4 == 0)
        hipLaunchKernelGGL((rmsnorm_pullback_kernel<TB, TX, 4>), grid, block, 0, stream, (const TB*)g_out, (const TX*)x,
                           (const TB*)weight, (const float*)g_residual, (float*)g_sum, (TB*)g_sum_branch, n_rows, P,
                           T_len, D, eps, res_bcast);
    else
        hipLaunchKernelGGL((rmsnorm_pullback_kernel<TB, TX, 1>), grid, block, 0, stream, (const TB*)g_out, (const TX*)x,
                           (const TB*)weight, (const float*)g_residual, (float*)g_sum, (TB*)g_sum_branch, n_rows, P,
                           T_len, D, eps, res_bcast);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

template <typename TB>
int launch_rmsnorm_x(int x_dtype, const void* g_out, const void* x, const void* weight, const void* g_residual,
                     void* g_sum, void* g_sum_branch, long long n_rows, int P, int T_len, int D, float eps,
                     int res_bcast, hipStream_t stream) {
    switch (x_dtype) {
        case LBI_F32: return launch_rmsnorm<TB, float>(g_out, x, weight, g_residual, g_sum, g_sum_branch, n_rows, P, T_len, D, eps, res_bcast, stream);
        case LBI_F16: return launch_rmsnorm<TB, _Float16>(g_out, x, weight, g_residual, g_sum, g_sum_branch, n_rows, P, T_len, D, eps, res_bcast, stream);
        default: return launch_rmsnorm<TB, bf16_raw>(g_out, x, weight, g_residual, g_sum, g_sum_branch, n_rows, P, T_len, D, eps, res_bcast, stream);
    }
}

template <typename T, int VEC>
int launch_gated_as(const void* g, const void* fc1, void* out, long long n_tokens, int P, int T_len, int hidden,
                    int g_bcast, hipStream_t stream) {
    if (n_tokens > 0x7fffffffLL) return fail(LBI_ERR_UNSUPPORTED, "lbi_gated_mlp_pullback: too many tokens");
    const int chunks = hidden / VEC;
    const int threads = chunks >= 256 ? 256 : ((chunks + 63) / 64) * 64;
    hipLaunchKernelGGL((gated_mlp_pullback_kernel<T, VEC>), dim3((unsigned)n_tokens), dim3(threads), 0, stream,
                       (const T*)g, (const T*)fc1, (T*)out, P, T_len, hidden, g_bcast);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

template <typename T>
int launch_gated(const void* g, const void* fc1, void* out, long long n_rows, int P, int T_len, int hidden,
                 int g_bcast, hipStream_t stream) {  // n_rows: tokens B * T
    constexpr int W = wide<T>();
    const bool aligned =
        (reinterpret_cast<uintptr_t>(g) | reinterpret_cast<uintptr_t>(fc1) | reinterpret_cast<uintptr_t>(out)) % 16 == 0;
    if (hidden % W == 0 && aligned) return launch_gated_as<T, W>(g, fc1, out, n_rows, P, T_len, hidden, g_bcast, stream);
    if (hidden % 4 == 0 && sizeof(T) == 4) return launch_gated_as<T, 4>(g, fc1, out, n_rows, P, T_len, hidden, g_bcast, stream);
    return launch_gated_as<T, 1>(g, fc1, out, n_rows, P, T_len, hidden, g_bcast, stream);
}

template <typename T>
int launch_qkv(const void* dq, const void* dk, const void* dv, const float* cos_t, const float* sin_t, void* out,
               long long n_rows, int T_len, int H, int Hkv, int Dh, int interleaved, hipStream_t stream) {
    const int half = Dh / 2;
    const int vec = half % 4 == 0 ? 4 : 1;
    const long long units = n_rows * (long long)(H + 2 * Hkv) * (half / vec);
    if (!fits_grid(units, 256)) return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_qkv_pullback: too many elements");
    const dim3 grid(blocks_for(units, 256)), block(256);
#define LBI_QKV_LAUNCH(VEC, IL)                                                                                       \
    hipLaunchKernelGGL((qkv_pullback_kernel<T, VEC, IL>), grid, block, 0, stream, (const T*)dq, (const T*)dk,        \
                       (const T*)dv, cos_t, sin_t, (T*)out, units, T_len, H, Hkv, Dh)
    if (vec == 4) {
        if (interleaved) LBI_QKV_LAUNCH(4, true); else LBI_QKV_LAUNCH(4, false);
    } else {
        if (interleaved) LBI_QKV_LAUNCH(1, true); else LBI_QKV_LAUNCH(1, false);
    }
#undef LBI_QKV_LAUNCH
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

template <typename T, int VEC, int KMAX, bool INTERLEAVED, bool EXACT>
int launch_qkv_conv_as(const void* dq, const void* dk, const void* dv, const float* cos_t, const float* sin_t,
                       const void* weight, void* out, long long n_seq, int T_len, int H, int Hkv, int Dh, int ksize,
                       hipStream_t stream) {
    constexpr int RUN = KMAX <= 4 ? 16 : 8;  // longer runs spill
    const long long units = n_seq * ((T_len + RUN - 1) / RUN) * (long long)(H + 2 * Hkv) * (Dh / 2 / VEC);
    if (!fits_grid(units, 256)) return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_qkv_conv_pullback: too many elements");
    hipLaunchKernelGGL((qkv_conv_pullback_kernel<T, VEC, KMAX, RUN, INTERLEAVED, EXACT>), dim3(blocks_for(units, 256)),
                       dim3(256), 0, stream, (const T*)dq, (const T*)dk, (const T*)dv, cos_t, sin_t, (const T*)weight,
                       (T*)out, units, T_len, H, Hkv, Dh, ksize);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

template <typename T, bool INTERLEAVED>
int launch_qkv_conv_il(const void* dq, const void* dk, const void* dv, const float* cos_t, const float* sin_t,
                       const void* weight, void* out, long long n_seq, int T_len, int H, int Hkv, int Dh, int ksize,
                       hipStream_t stream) {
    const bool vec = (Dh / 2) % 4 == 0;
    // the 4 x 4 weights of a channel group are contiguous; 4-element loads of them need 4-element alignment
    const bool exact = vec && ksize == 4 && reinterpret_cast<uintptr_t>(weight) % (4 * sizeof(T)) == 0;
    if (exact)
        return launch_qkv_conv_as<T, 4, 4, INTERLEAVED, true>(dq, dk, dv, cos_t, sin_t, weight, out, n_seq, T_len, H, Hkv, Dh, ksize, stream);
    if (vec && ksize <= 4)
        return launch_qkv_conv_as<T, 4, 4, INTERLEAVED, false>(dq, dk, dv, cos_t, sin_t, weight, out, n_seq, T_len, H, Hkv, Dh, ksize, stream);
    if (vec)
        return launch_qkv_conv_as<T, 4, 8, INTERLEAVED, false>(dq, dk, dv, cos_t, sin_t, weight, out, n_seq, T_len, H, Hkv, Dh, ksize, stream);
    if (ksize <= 4)
        return launch_qkv_conv_as<T, 1, 4, INTERLEAVED, false>(dq, dk, dv, cos_t, sin_t, weight, out, n_seq, T_len, H, Hkv, Dh, ksize, stream);
    return launch_qkv_conv_as<T, 1, 8, INTERLEAVED, false>(dq, dk, dv, cos_t, sin_t, weight, out, n_seq, T_len, H, Hkv, Dh, ksize, stream);
}

template <typename T>
int launch_qkv_conv(const void* dq, const void* dk, const void* dv, const float* cos_t, const float* sin_t,
                    const void* weight, void* out, long long n_seq, int T_len, int H, int Hkv, int Dh, int interleaved,
                    int ksize, hipStream_t stream) {
    if (interleaved)
        return launch_qkv_conv_il<T, true>(dq, dk, dv, cos_t, sin_t, weight, out, n_seq, T_len, H, Hkv, Dh, ksize, stream);
    return launch_qkv_conv_il<T, false>(dq, dk, dv, cos_t, sin_t, weight, out, n_seq, T_len, H, Hkv, Dh, ksize, stream);
}

template <typename T, int VEC, int KMAX, int RUN, bool EXACT = false>
int launch_conv_as(const void* g_out, const void* weight, void* g_in, long long n_seq, int T_len, int C, int ksize,
                   hipStream_t stream) {
    const long long units = n_seq * ((T_len + RUN - 1) / RUN) * (C / VEC);
    if (!fits_grid(units, 256)) return fail(LBI_ERR_UNSUPPORTED, "lbi_causal_conv1d_pullback: too many elements");
    hipLaunchKernelGGL((causal_conv1d_pullback_kernel<T, VEC, KMAX, RUN, EXACT>), dim3(blocks_for(units, 256)), dim3(256), 0,
                       stream, (const T*)g_out, (const T*)weight, (T*)g_in, units, T_len, C, ksize);
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

template <typename T>
int launch_conv(const void* g_out, const void* weight, void* g_in, long long n_seq, int T_len, int C, int ksize,
                hipStream_t stream) {
    constexpr int W = wide<T>();
    const bool aligned = (reinterpret_cast<uintptr_t>(g_out) | reinterpret_cast<uintptr_t>(g_in)) % 16 == 0;
    if (C % W == 0 && aligned) {
        if (ksize == 4 && reinterpret_cast<uintptr_t>(weight) % 16 == 0)
            return launch_conv_as<T, W, 4, 8, true>(g_out, weight, g_in, n_seq, T_len, C, ksize, stream);
        if (ksize <= 4) return launch_conv_as<T, W, 4, 8>(g_out, weight, g_in, n_seq, T_len, C, ksize, stream);
        if (ksize <= 8) return launch_conv_as<T, W, 8, 8>(g_out, weight, g_in, n_seq, T_len, C, ksize, stream);
    }
    if (ksize <= 4) return launch_conv_as<T, 1, 4, 8>(g_out, weight, g_in, n_seq, T_len, C, ksize, stream);
    if (ksize <= 8) return launch_conv_as<T, 1, 8, 8>(g_out, weight, g_in, n_seq, T_len, C, ksize, stream);
    if (ksize <= 16) return launch_conv_as<T, 1, 16, 4>(g_out, weight, g_in, n_seq, T_len, C, ksize, stream);
    return launch_conv_as<T, 1, 64, 1>(g_out, weight, g_in, n_seq, T_len, C, ksize, stream);
}

inline bool valid_dtype(int dtype) { return dtype == LBI_F32 || dtype == LBI_F16 || dtype == LBI_BF16; }
inline bool positive_int(int64_t v) { return v > 0 && v <= 0x7fffffff; }

}  // namespace region
}  // namespace lbi

using namespace lbi;

extern "C" int lbi_rmsnorm_pullback(const void* g_out, const void* x, const void* weight, const void* g_residual,
                                    void* g_sum, void* g_sum_branch, int64_t B, int64_t P, int64_t T, int64_t D,
                                    float eps, int g_residual_broadcast_t, int branch_dtype, int x_dtype,
                                    void* stream) {
    clear_error();
    if (!g_out || !x || !weight) return fail(LBI_ERR_INVALID, "lbi_rmsnorm_pullback: null input pointer");
    if (!g_sum && !g_sum_branch) return fail(LBI_ERR_INVALID, "lbi_rmsnorm_pullback: no output requested");
    if (!region::valid_dtype(branch_dtype) || !region::valid_dtype(x_dtype))
        return fail(LBI_ERR_INVALID, "lbi_rmsnorm_pullback: bad dtype");
    if (B < 0 || P < 0 || T < 0 || !region::positive_int(D) || P > 0x7fffffff || T > 0x7fffffff)
        return fail(LBI_ERR_INVALID, "lbi_rmsnorm_pullback: bad size B=%lld P=%lld T=%lld D=%lld", (long long)B,
                    (long long)P, (long long)T, (long long)D);
    const long long n_rows = (long long)B * P * T;
    if (n_rows == 0) return LBI_OK;
    if (!region::fits_grid(n_rows, 4)) return fail(LBI_ERR_UNSUPPORTED, "lbi_rmsnorm_pullback: too many rows");
    if (g_residual_broadcast_t && g_sum == g_residual)
        return fail(LBI_ERR_INVALID, "lbi_rmsnorm_pullback: a residual shared over T cannot be updated in place");
    const int rb = g_residual_broadcast_t != 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (branch_dtype) {
        case LBI_F32: return region::launch_rmsnorm_x<float>(x_dtype, g_out, x, weight, g_residual, g_sum, g_sum_branch, n_rows, (int)P, (int)T, (int)D, eps, rb, s);
        case LBI_F16: return region::launch_rmsnorm_x<_Float16>(x_dtype, g_out, x, weight, g_residual, g_sum, g_sum_branch, n_rows, (int)P, (int)T, (int)D, eps, rb, s);
        default: return region::launch_rmsnorm_x<bf16_raw>(x_dtype, g_out, x, weight, g_residual, g_sum, g_sum_branch, n_rows, (int)P, (int)T, (int)D, eps, rb, s);
    }
}

extern "C" int lbi_gated_mlp_pullback(const void* g_down_input, const void* fc1_output, void* g_fc1_output, int64_t B,
                                      int64_t P, int64_t T, int64_t hidden, int g_broadcast_t, int dtype,
                                      void* stream) {
    clear_error();
    if (!g_down_input || !fc1_output || !g_fc1_output)
        return fail(LBI_ERR_INVALID, "lbi_gated_mlp_pullback: null pointer");
    if (!region::valid_dtype(dtype)) return fail(LBI_ERR_INVALID, "lbi_gated_mlp_pullback: bad dtype %d", dtype);
    if (B < 0 || P < 0 || T < 0 || !region::positive_int(hidden) || P > 0x7fffffff || T > 0x7fffffff)
        return fail(LBI_ERR_INVALID, "lbi_gated_mlp_pullback: bad size");
    if (B == 0 || P == 0 || T == 0) return LBI_OK;
    const long long n_rows = (long long)B * T;  // one workgroup per token
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case LBI_F32: return region::launch_gated<float>(g_down_input, fc1_output, g_fc1_output, n_rows, (int)P, (int)T, (int)hidden, g_broadcast_t != 0, s);
        case LBI_F16: return region::launch_gated<_Float16>(g_down_input, fc1_output, g_fc1_output, n_rows, (int)P, (int)T, (int)hidden, g_broadcast_t != 0, s);
        default: return region::launch_gated<bf16_raw>(g_down_input, fc1_output, g_fc1_output, n_rows, (int)P, (int)T, (int)hidden, g_broadcast_t != 0, s);
    }
}

extern "C" int lbi_attn_heads_split(const void* g_merged, void* g_heads, int64_t B, int64_t P, int64_t T, int64_t H,
                                    int64_t Dh, int dtype, void* stream) {
    clear_error();
    if (!g_merged || !g_heads) return fail(LBI_ERR_INVALID, "lbi_attn_heads_split: null pointer");
    if (!region::valid_dtype(dtype)) return fail(LBI_ERR_INVALID, "lbi_attn_heads_split: bad dtype %d", dtype);
    if (B < 0 || P < 0 || !region::positive_int(T) || !region::positive_int(H) || !region::positive_int(Dh))
        return fail(LBI_ERR_INVALID, "lbi_attn_heads_split: bad size");
    const long long n = (long long)B * P;
    if (n == 0) return LBI_OK;
    const size_t head_bytes = (size_t)Dh * dtype_size(dtype);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool aligned = (reinterpret_cast<uintptr_t>(g_merged) | reinterpret_cast<uintptr_t>(g_heads)) % 16 == 0;
    if (head_bytes % 16 == 0 && aligned) {
        typedef unsigned int chunk16 __attribute__((ext_vector_type(4)));
        const int cph = (int)(head_bytes / 16);
        const long long chunks = n * T * H * cph;
        if (!region::fits_grid(chunks, 256)) return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_heads_split: too many elements");
        hipLaunchKernelGGL((region::heads_split_kernel<chunk16>), dim3(region::blocks_for(chunks, 256)), dim3(256), 0, s,
                           (const chunk16*)g_merged, (chunk16*)g_heads, chunks, (int)T, (int)H, cph);
    } else if (dtype == LBI_F32) {
        const long long chunks = n * T * H * Dh;
        if (!region::fits_grid(chunks, 256)) return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_heads_split: too many elements");
        hipLaunchKernelGGL((region::heads_split_kernel<unsigned int>), dim3(region::blocks_for(chunks, 256)), dim3(256), 0,
                           s, (const unsigned int*)g_merged, (unsigned int*)g_heads, chunks, (int)T, (int)H, (int)Dh);
    } else {
        const long long chunks = n * T * H * Dh;
        if (!region::fits_grid(chunks, 256)) return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_heads_split: too many elements");
        hipLaunchKernelGGL((region::heads_split_kernel<unsigned short>), dim3(region::blocks_for(chunks, 256)), dim3(256),
                           0, s, (const unsigned short*)g_merged, (unsigned short*)g_heads, chunks, (int)T, (int)H,
                           (int)Dh);
    }
    LBI_HIP_CHECK(hipGetLastError());
    return LBI_OK;
}

extern "C" int lbi_attn_qkv_pullback(const void* dq, const void* dk, const void* dv, const float* rope_cos,
                                     const float* rope_sin, void* g_qkv, int64_t B, int64_t P, int64_t T, int64_t H,
                                     int64_t Hkv, int64_t Dh, int interleaved, int dtype, void* stream) {
    clear_error();
    if (!dq || !dk || !dv || !rope_cos || !rope_sin || !g_qkv)
        return fail(LBI_ERR_INVALID, "lbi_attn_qkv_pullback: null pointer");
    if (!region::valid_dtype(dtype)) return fail(LBI_ERR_INVALID, "lbi_attn_qkv_pullback: bad dtype %d", dtype);
    if (B < 0 || P < 0 || !region::positive_int(T) || !region::positive_int(H) || !region::positive_int(Hkv) ||
        !region::positive_int(Dh))
        return fail(LBI_ERR_INVALID, "lbi_attn_qkv_pullback: bad size");
    if (H % Hkv != 0) return fail(LBI_ERR_INVALID, "lbi_attn_qkv_pullback: H=%lld not a multiple of Hkv=%lld", (long long)H, (long long)Hkv);
    if (Dh % 2 != 0) return fail(LBI_ERR_INVALID, "lbi_attn_qkv_pullback: rotary embedding needs an even head dim, got %lld", (long long)Dh);
    const long long n_rows = (long long)B * P * T;
    if (n_rows == 0) return LBI_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case LBI_F32: return region::launch_qkv<float>(dq, dk, dv, rope_cos, rope_sin, g_qkv, n_rows, (int)T, (int)H, (int)Hkv, (int)Dh, interleaved != 0, s);
        case LBI_F16: return region::launch_qkv<_Float16>(dq, dk, dv, rope_cos, rope_sin, g_qkv, n_rows, (int)T, (int)H, (int)Hkv, (int)Dh, interleaved != 0, s);
        default: return region::launch_qkv<bf16_raw>(dq, dk, dv, rope_cos, rope_sin, g_qkv, n_rows, (int)T, (int)H, (int)Hkv, (int)Dh, interleaved != 0, s);
    }
}

extern "C" int lbi_attn_qkv_conv_pullback(const void* dq, const void* dk, const void* dv, const float* rope_cos,
                                          const float* rope_sin, const void* conv_weight, void* g_in, int64_t B,
                                          int64_t P, int64_t T, int64_t H, int64_t Hkv, int64_t Dh, int interleaved,
                                          int64_t ksize, int dtype, void* stream) {
    clear_error();
    if (!dq || !dk || !dv || !rope_cos || !rope_sin || !conv_weight || !g_in)
        return fail(LBI_ERR_INVALID, "lbi_attn_qkv_conv_pullback: null pointer");
    if (!region::valid_dtype(dtype)) return fail(LBI_ERR_INVALID, "lbi_attn_qkv_conv_pullback: bad dtype %d", dtype);
    if (B < 0 || P < 0 || !region::positive_int(T) || !region::positive_int(H) || !region::positive_int(Hkv) ||
        !region::positive_int(Dh) || (long long)(H + 2 * Hkv) * Dh > 0x7fffffffLL)
        return fail(LBI_ERR_INVALID, "lbi_attn_qkv_conv_pullback: bad size");
    if (H % Hkv != 0) return fail(LBI_ERR_INVALID, "lbi_attn_qkv_conv_pullback: H=%lld not a multiple of Hkv=%lld", (long long)H, (long long)Hkv);
    if (Dh % 2 != 0) return fail(LBI_ERR_INVALID, "lbi_attn_qkv_conv_pullback: rotary embedding needs an even head dim, got %lld", (long long)Dh);
    if (ksize < 1) return fail(LBI_ERR_INVALID, "lbi_attn_qkv_conv_pullback: bad filter length %lld", (long long)ksize);
    if (ksize > 8)
        return fail(LBI_ERR_UNSUPPORTED, "lbi_attn_qkv_conv_pullback: filter length %lld above 8; call lbi_attn_qkv_pullback and lbi_causal_conv1d_pullback", (long long)ksize);
    const long long n_seq = (long long)B * P;
    if (n_seq == 0) return LBI_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case LBI_F32: return region::launch_qkv_conv<float>(dq, dk, dv, rope_cos, rope_sin, conv_weight, g_in, n_seq, (int)T, (int)H, (int)Hkv, (int)Dh, interleaved != 0, (int)ksize, s);
        case LBI_F16: return region::launch_qkv_conv<_Float16>(dq, dk, dv, rope_cos, rope_sin, conv_weight, g_in, n_seq, (int)T, (int)H, (int)Hkv, (int)Dh, interleaved != 0, (int)ksize, s);
        default: return region::launch_qkv_conv<bf16_raw>(dq, dk, dv, rope_cos, rope_sin, conv_weight, g_in, n_seq, (int)T, (int)H, (int)Hkv, (int)Dh, interleaved != 0, (int)ksize, s);
    }
}

extern "C" int lbi_causal_conv1d_pullback(const void* g_out, const void* weight, void* g_in, int64_t N, int64_t T,
                                          int64_t C, int64_t ksize, int dtype, void* stream) {
    clear_error();
    if (!g_out || !weight || !g_in) return fail(LBI_ERR_INVALID, "lbi_causal_conv1d_pullback: null pointer");
    if (g_out == g_in) return fail(LBI_ERR_INVALID, "lbi_causal_conv1d_pullback: in-place call not supported");
    if (!region::valid_dtype(dtype)) return fail(LBI_ERR_INVALID, "lbi_causal_conv1d_pullback: bad dtype %d", dtype);
    if (N < 0 || !region::positive_int(T) || !region::positive_int(C) || ksize < 1 || ksize > 64)
        return fail(LBI_ERR_INVALID, "lbi_causal_conv1d_pullback: bad size");
    if (N == 0) return LBI_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
        case LBI_F32: return region::launch_conv<float>(g_out, weight, g_in, N, (int)T, (int)C, (int)ksize, s);
        case LBI_F16: return region::launch_conv<_Float16>(g_out, weight, g_in, N, (int)T, (int)C, (int)ksize, s);
        default: return region::launch_conv<bf16_raw>(g_out, weight, g_in, N, (int)T, (int)C, (int)ksize, s);
    }
}
