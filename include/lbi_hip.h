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
 * aligned; its contents on entry are ignored.  Replaces
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

#ifdef __cplusplus
}
#endif

#endif /* LBI_HIP_H */
