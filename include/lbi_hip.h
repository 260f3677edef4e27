/*
 * lbi_hip.h - C ABI of liblbi_hip.so, the gfx950 (MI355X) kernels of the LBI
 * bounded-interface backward hot path.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void* so the header needs no HIP include), launches on that
 * stream without synchronising the host, never allocates or frees device
 * memory, never writes to its inputs, and returns 0 on success or a negative
 * lbi_status.  After a failure lbi_last_error() returns a message for the
 * calling thread.  All tensors are dense, row-major and contiguous.
 *
 * "reference" below is shaunlee8/latent-bounded-interfaces.
 */
#ifndef LBI_HIP_H
#define LBI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element types of device buffers. */
enum lbi_dtype {
    LBI_F32 = 0,
    LBI_F16 = 1,
    LBI_BF16 = 2
};

enum lbi_status {
    LBI_OK = 0,
    LBI_ERR_INVALID = -1,     /* contract violation: null pointer, bad size, bad dtype        */
    LBI_ERR_UNSUPPORTED = -2, /* valid request this build has no kernel for                    */
    LBI_ERR_HIP = -3,         /* a HIP runtime call or launch failed; message carries the text */
    LBI_ERR_WORKSPACE = -4    /* workspace buffer missing or smaller than *_workspace_bytes()  */
};

/* ABI revision; bumped whenever a signature below changes. */
int lbi_abi_version(void);

/* Message of the last failure on the calling thread ("" if none). */
const char* lbi_last_error(void);

/*
 * Suffix scan of per-region interface pullback matrices.
 *
 *   mats [B, K, d, d] (in_dtype)  ->  out [B, K+1, d, d] (out_dtype, LBI_F32 only)
 *   out[b, r] = mats[b, r] @ mats[b, r+1] @ ... @ mats[b, K-1]   (r < K),   out[b, K] = I
 *
 * Products are accumulated in fp32 whatever in_dtype is.  K == 0 is valid and
 * yields the identity.  Replaces the native entry suffix_scan_mats of the
 * reference (cuda/interface/binding.cpp:5-11, launcher
 * cuda/interface/suffix_scan.cu:70-115) behind
 * suffix_scan_pullbacks (cuda/interface/__init__.py:33-36).
 */
int lbi_suffix_scan(const void* mats, void* out,
                    int64_t B, int64_t K, int64_t d,
                    int in_dtype, int out_dtype, void* stream);

/*
 * Suffix scan and cotangent chain in one pass over mats:
 *
 *   out as lbi_suffix_scan;  cot [B, K+1, d] (fp32) as lbi_suffix_cotangents for g [B, d] (fp32).
 *
 * This is the whole of propagate_state_adjoint_with_jacobian_scan of the reference
 * (backward/suffix_scan.py:41-56: scan, then K mat-vecs suffix[r] @ g), with the mat-vecs
 * computed as the chain cot[r] = mats[r] @ cot[r+1] from the operand registers of the
 * matrix products, i.e. at no extra memory traffic.
 */
int lbi_suffix_scan_with_cotangents(const void* mats, const void* g, void* out, void* cot,
                                    int64_t B, int64_t K, int64_t d,
                                    int in_dtype, int out_dtype, void* stream);

/*
 * Both scan entries above with one more argument.  g and cot are both given (as lbi_suffix_scan_with_cotangents) or
 * both null (as lbi_suffix_scan).  flags: 0, or LBI_SCAN_EXACT_SUFFIX.
 *
 * With bf16 storage at d = 256 the products run on the 16-bit matrix cores: the stored matrix enters as it is, the
 * running suffix (fp32) as a sum of bf16 planes, accumulation is fp32.  By default the suffix operand is rounded to
 * 16 significand bits (two planes: 256 times finer than the rounding of the stored inputs themselves; measured
 * error against fp64 at K = 128 below 2e-4 of the largest entry, where the bar for 16-bit storage is 2e-2
 * against the fp32 path); LBI_SCAN_EXACT_SUFFIX keeps its exact fp32 value (three planes, half again as many
 * products): what is left is the rounding of the fp32 accumulation (measured <= 1.2e-5 at K = 128, <= 1e-5 on
 * shorter chains).  The flag changes nothing for fp32 and fp16 storage or other
 * widths, whose products are fp32 throughout.  The reference's native scan has one precision
 * (cuda/interface/suffix_scan.cu:76-110: fp32 SGEMM, which its own tests allow TF32-sized errors,
 * tests/test_interface_scan.py:34-39).
 */
enum lbi_scan_flags {
    LBI_SCAN_EXACT_SUFFIX = 1
};

int lbi_suffix_scan_ex(const void* mats, const void* g, void* out, void* cot,
                       int64_t B, int64_t K, int64_t d,
                       int in_dtype, int out_dtype, int flags, void* stream);

/*
 * Cotangent-only suffix chain: no d x d product is formed.
 *
 *   mats [B, K, d, d] (in_dtype), g [B, d] (fp32)  ->  out [B, K+1, d] (fp32)
 *   out[b, K] = g[b],   out[b, r] = mats[b, r] @ out[b, r+1]
 *
 * Equals suffix[r] @ g of propagate_state_adjoint_with_jacobian_scan
 * (reference backward/suffix_scan.py:41-56) and the sequential chain of
 * reference backward/scan.py:63-72, computed with one pass over mats.
 */
int lbi_suffix_cotangents(const void* mats, const void* g, void* out,
                          int64_t B, int64_t K, int64_t d,
                          int in_dtype, void* stream);

/*
 * Suffix matrices applied to the terminal cotangent, all of them in one launch:
 *
 *   suffix [B, M, d, d] (fp32), g [B, d] (fp32)  ->  out [B, M, d] (fp32),   out[b, r] = suffix[b, r] @ g[b]
 *
 * The K mat-vecs apply_jacobian_t(suffix[r], g) of propagate_state_adjoint_with_jacobian_scan in the reference
 * (backward/suffix_scan.py:49-53, :24-38), on the result of lbi_suffix_scan (M = K + 1 covers the identity tail,
 * which returns g itself).  With the chain cotangents of lbi_suffix_scan_with_cotangents it gives the two sides of
 * the reference's per-step cross-check interface_scan_rms (backward/scan.py:63-72).
 */
int lbi_suffix_apply(const void* suffix, const void* g, void* out,
                     int64_t B, int64_t M, int64_t d, void* stream);

/*
 * Attention input-pullback for P cotangent basis directions at once.
 *
 *   q, k, v [B, H, T, Dh],  d_out [B, P, H, T, Dh]   (dtype)
 *   -> dq, dk, dv [B, P, H, T, Dh]                    (dtype)
 *
 *   Pm = softmax(scale * q k^T + causal mask);  dv_p = Pm^T d_out_p;
 *   dP_p = d_out_p v^T;  delta_p = rowsum(dP_p * Pm);  dS_p = Pm * (dP_p - delta_p);
 *   dq_p = scale * dS_p k;  dk_p = scale * dS_p^T q.
 *
 * Storage dtype is LBI_F16, LBI_BF16 or LBI_F32; accumulation is fp32.  The
 * softmax statistics are recomputed inside (no forward output or logsumexp is
 * taken from the caller).  `workspace` must hold at least
 * lbi_attn_pullback_workspace_bytes(...) bytes of device memory, 256-byte
 * aligned; its contents on entry are ignored.  That size is 0 for short
 * sequences (16-bit storage, any T up to 256 at Dh = 64 and up
 * to 128 at Dh = 128), which run as a single launch; `workspace` may then be
 * null.  Replaces
 * attention_input_pullback_basis_simple / _mma_p1 / _mma_pblock4 of the
 * reference (cuda/transformer/binding.cpp:6-22; kernels
 * cuda/transformer/attention_pullback_mma.cu:60-321,
 * cuda/transformer/attention_pullback_simple.cu:132-330) behind
 * attention_input_pullback_basis (cuda/transformer/__init__.py:279-355),
 * together with the flash forward the reference wrapper re-runs to get the
 * softmax statistics (cuda/transformer/__init__.py:248-256).
 */
size_t lbi_attn_pullback_workspace_bytes(int64_t B, int64_t H, int64_t T, int64_t Dh,
                                         int64_t P, int dtype);

int lbi_attn_pullback(const void* q, const void* k, const void* v, const void* d_out,
                      void* dq, void* dk, void* dv,
                      void* workspace, size_t workspace_bytes,
                      int64_t B, int64_t H, int64_t T, int64_t Dh, int64_t P,
                      float softmax_scale, int causal, int dtype, void* stream);

/*
 * lbi_attn_pullback without a workspace argument and without any allocation: the scratch memory (softmax
 * statistics, -delta, the fp32 forward output) lives in a static device array of
 * LBI_ATTN_STATIC_SCRATCH_BYTES inside the library, one copy per GPU, held until the process ends.
 *
 * This entry has no counterpart in the reference.  It is for callers that cannot allocate device memory:
 * code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Arguments and results
 * are those of lbi_attn_pullback (the same kernels run, results are bit-identical).  A call whose
 * lbi_attn_pullback_workspace_bytes(...) exceeds LBI_ATTN_STATIC_SCRATCH_BYTES returns LBI_ERR_WORKSPACE.
 * All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different streams or
 * threads) race on it; serialise them.
 *
 * Runtime calls it makes: hipGetDevice on every call; on the FIRST call per device also hipGetSymbolAddress
 * (the array's address on that device, kept afterwards) and, for kernels that need more than 64 KiB of LDS,
 * hipFuncSetAttribute once per kernel and device.  None of these allocates, but the first-call ones must not
 * happen for the first time inside a stream capture: make one call of the same shape outside the capture first
 * (a warm-up), then capture; captured and later calls only launch kernels.
 */
#define LBI_ATTN_STATIC_SCRATCH_BYTES (32u << 20)

int lbi_attn_pullback_static(const void* q, const void* k, const void* v, const void* d_out,
                             void* dq, void* dk, void* dv,
                             int64_t B, int64_t H, int64_t T, int64_t Dh, int64_t P,
                             float softmax_scale, int causal, int dtype, void* stream);

/*
 * Region-level input pullback of a Transformer block (the pieces around the matrix products,
 * which the caller issues as plain GEMMs, and around lbi_attn_pullback).  Together they
 * implement TransformerLowering.input_pullback_basis of the reference
 * (backends/transformer.py:64-75; stub backends/transformer_cuda.py:45-64) for the block
 * of backends/transformer.py:118-215.  Cotangent tensors carry a basis axis: [B, P, T, *];
 * forward activations are [B, T, *] and are shared by the P directions.
 */

/*
 * RMSNorm pullback, optionally fused with the residual-stream add.
 *
 *   y = (x_r * rsqrt(mean(x_r^2) + eps)) * weight,   x_r = x rounded to branch_dtype
 *   g_x = r * (weight o g_out) - x_r * r^3 * mean(x_r o weight o g_out)
 *   out = g_x + g_residual            (g_residual may be NULL = 0)
 *
 *   g_out [B,P,T,D] and weight [D] in branch_dtype; x [B,T,D] in x_dtype (the pre-norm
 *   residual stream, reference backends/transformer.py:197,201);
 *   g_residual [B,P,T,D] fp32 or NULL; outputs g_sum [B,P,T,D] fp32 and/or g_sum_branch
 *   [B,P,T,D] branch_dtype (either may be NULL, not both).  g_sum may alias g_residual.
 *   g_residual_broadcast_t != 0: g_residual is [B,P,D], the same for every position (the
 *   cotangent a mean-pooling interface sends into the region output, reference
 *   interfaces/vector_mlp.py:111-116); it then must not alias g_sum.
 *   Forward: RMSNorm.forward, reference backbones/transformer/block.py:12-23, applied by
 *   TransformerBlock._prenorm (block.py:66-76).
 */
int lbi_rmsnorm_pullback(const void* g_out, const void* x, const void* weight, const void* g_residual,
                         void* g_sum, void* g_sum_branch,
                         int64_t B, int64_t P, int64_t T, int64_t D, float eps,
                         int g_residual_broadcast_t, int branch_dtype, int x_dtype, void* stream);

/*
 * Gated-MLP pullback through  down_input = up * silu(gate),  [up | gate] = fc1_output.
 *
 *   g_down_input [B,P,T,hidden], fc1_output [B,T,2*hidden]  ->  g_fc1_output [B,P,T,2*hidden]
 *   g_up = g * silu(gate);   g_gate = g * up * silu'(gate)
 *   g_broadcast_t != 0: g_down_input is [B,P,hidden], the same for every position.
 *
 * Forward: reference backends/transformer.py:172-176 (GatedMLP.forward,
 * backbones/transformer/mlp.py:30-32).
 */
int lbi_gated_mlp_pullback(const void* g_down_input, const void* fc1_output, void* g_fc1_output,
                           int64_t B, int64_t P, int64_t T, int64_t hidden,
                           int g_broadcast_t, int dtype, void* stream);

/*
 * Head split of the out_proj-input cotangent: [B,P,T,H*Dh] -> [B,P,H,T,Dh], the layout
 * lbi_attn_pullback takes as d_out (transpose of reference backends/transformer.py:152-153).
 */
int lbi_attn_heads_split(const void* g_merged, void* g_heads,
                         int64_t B, int64_t P, int64_t T, int64_t H, int64_t Dh, int dtype, void* stream);

/*
 * Cotangent of the packed q/k/v projection from the outputs of lbi_attn_pullback.
 *
 *   dq, dk, dv [B,P,H,T,Dh]  ->  g_qkv [B,P,T,(H + 2*Hkv)*Dh]
 *   q part: transposed rotary embedding of dq;  k part: the same of the sum of dk over the
 *   H/Hkv query heads that share a key head;  v part: that sum of dv.
 *   rope_cos, rope_sin [T, Dh/2] fp32: cos and sin of position * base^(-2i/Dh).
 *
 * Transposes reference backends/transformer.py:124-132 (split, head views, apply_rope of
 * backbones/transformer/rope.py:6-34 in its half-split or interleaved pairing, and
 * CausalSelfAttention._expand_kv, backbones/transformer/attention.py:61-65).
 */
int lbi_attn_qkv_pullback(const void* dq, const void* dk, const void* dv,
                          const float* rope_cos, const float* rope_sin, void* g_qkv,
                          int64_t B, int64_t P, int64_t T, int64_t H, int64_t Hkv, int64_t Dh,
                          int interleaved, int dtype, void* stream);

/*
 * Pullback of the depthwise causal convolution applied to the packed projection
 * (reference backends/transformer.py:121-122: Conv1d(groups=C, padding=k-1), first T outputs).
 *
 *   g_out [N,T,C], weight [C,k]  ->  g_in [N,T,C],   N = B*P
 *   g_in[n,s,c] = sum_i weight[c,k-1-i] * g_out[n,s+i,c]   over s+i < T
 */
int lbi_causal_conv1d_pullback(const void* g_out, const void* weight, void* g_in,
                               int64_t N, int64_t T, int64_t C, int64_t ksize, int dtype, void* stream);

/*
 * lbi_attn_qkv_pullback followed by lbi_causal_conv1d_pullback in one pass, without storing the
 * cotangent of the convolved projection (reference backends/transformer.py:121-132 transposed):
 *
 *   dq, dk, dv [B,P,H,T,Dh], conv_weight [(H + 2*Hkv)*Dh, k]  ->  g_in [B,P,T,(H + 2*Hkv)*Dh]
 *
 * The intermediate is rounded to the storage type as the two calls would store it and the sums run
 * in the same order: fp32 results are bit-identical to theirs, 16-bit results equal up to the last
 * place of a final rounding.  k <= 8; longer filters return LBI_ERR_UNSUPPORTED and take the two
 * calls.
 */
int lbi_attn_qkv_conv_pullback(const void* dq, const void* dk, const void* dv,
                               const float* rope_cos, const float* rope_sin, const void* conv_weight,
                               void* g_in, int64_t B, int64_t P, int64_t T, int64_t H, int64_t Hkv,
                               int64_t Dh, int interleaved, int64_t ksize, int dtype, void* stream);

/*
 * Parameter gradients of a Transformer block that are not matrix products (the others are plain GEMMs of a
 * module's output cotangent with its cached input).  Part of TransformerLowering.parameter_vjp of the reference
 * (backends/transformer.py:76-85; autograd version :332-355, which gets them from torch.autograd.grad).
 * Sums run in a fixed order (per-workgroup partial sums in `workspace`, added in workgroup order): reruns are
 * bit-identical.  Results are fp32.
 *
 * RMSNorm weight:  weight_grad[c] = sum over rows of g_out[row,c] * round(x_r[row,c] * rsqrt(mean_c(x_r^2) + eps)),
 *   x_r = x rounded to `dtype` (RMSNorm.forward, reference backbones/transformer/block.py:12-23).
 *   g_out [rows,D] in `dtype` (the weight's), x [rows,D] in `x_dtype` (= dtype, or fp32 for an fp32 residual
 *   stream); D a multiple of 4, at most 2048.  workspace: lbi_rmsnorm_weight_grad_workspace_bytes(rows, D) bytes,
 *   16-byte aligned.
 */
size_t lbi_rmsnorm_weight_grad_workspace_bytes(int64_t rows, int64_t D);
int lbi_rmsnorm_weight_grad(const void* g_out, const void* x, float* weight_grad,
                            void* workspace, size_t workspace_bytes,
                            int64_t rows, int64_t D, float eps, int dtype, int x_dtype, void* stream);

/*
 * Depthwise causal convolution (reference backends/transformer.py:121-122: Conv1d(groups=C, padding=k-1),
 * first T outputs), weight and bias gradient:
 *   grads[c*k + j]   = sum over b, t >= k-1-j of g_out[b,t,c] * x[b, t-(k-1-j), c]      (weight [C,1,k])
 *   grads[C*k + c]   = sum over b, t of g_out[b,t,c]                                    (bias [C])
 *   g_out, x [B,T,C] in `dtype`; k <= 8.  workspace: lbi_causal_conv1d_weight_grad_workspace_bytes(B,T,C,k) bytes.
 */
size_t lbi_causal_conv1d_weight_grad_workspace_bytes(int64_t B, int64_t T, int64_t C, int64_t ksize);
int lbi_causal_conv1d_weight_grad(const void* g_out, const void* x, float* grads,
                                  void* workspace, size_t workspace_bytes,
                                  int64_t B, int64_t T, int64_t C, int64_t ksize, int dtype, void* stream);

/*
 * Frobenius and spectral (largest singular value) norms of N square matrices, the per-step Jacobian
 * diagnostics of the interface scan (reference backward/suffix_scan.py:105-134, which calls
 * torch.linalg.matrix_norm with ord="fro" and ord=2, a singular value decomposition per matrix).
 *
 *   mats [N,d,d] (dtype)  ->  spectral [N], frobenius [N]   (fp32)
 *
 * No decomposition: the top eigenvalue of A^T A comes from repeated squaring with the trace divided
 * out, at most 24 squarings, which bounds the relative error by 2^-25 log(d) plus fp32 rounding for
 * any spectrum.  `workspace` must hold lbi_matrix_norms_workspace_bytes(N, d) bytes (0 for d <= 88,
 * whose buffers fit in LDS; larger matrices run their products on the fp32 matrix cores out of the
 * workspace), 16-byte aligned.  d <= 2048.
 */
size_t lbi_matrix_norms_workspace_bytes(int64_t N, int64_t d);
int lbi_matrix_norms(const void* mats, float* spectral, float* frobenius,
                     void* workspace, size_t workspace_bytes,
                     int64_t N, int64_t d, int dtype, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* LBI_HIP_H */
