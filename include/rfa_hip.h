/*
 * rfa_hip.h -- C ABI of librfa_hip.so, the MI355X (gfx950) kernel library for
 * Random Feature Attention.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer on the current HIP device unless said
 *     otherwise; fp16 tensors are IEEE binary16, contiguous, 16-byte aligned;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     all work is enqueued on it and nothing is synchronised;
 *   - functions return RFA_OK (0) or a negative RFA_ERR_* code; the message for
 *     the last error on the calling thread is returned by rfa_last_error();
 *   - nothing is allocated by the library: kernels that need scratch memory
 *     take a caller-owned workspace whose size the matching *_workspace_bytes
 *     function reports (0 is a valid answer; then workspace may be NULL);
 *   - K = 2 * proj_dim is the width of the feature vectors phi(q), phi(k);
 *     d = head_dim; N = bsz * num_heads.
 *
 * Each entry point cites the reference interface it replaces
 * (paths relative to the Noahs-ARK/RFA repository root).
 */
#ifndef RFA_HIP_H
#define RFA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RFA_OK 0
#define RFA_ERR_NULL_POINTER (-1)  /* a required pointer is NULL              */
#define RFA_ERR_BAD_SHAPE (-2)     /* negative / inconsistent sizes           */
#define RFA_ERR_UNSUPPORTED (-3)   /* (K, d) combination has no kernel        */
#define RFA_ERR_ALIGNMENT (-4)     /* a pointer is not 16-byte aligned        */
#define RFA_ERR_WORKSPACE (-5)     /* workspace missing or too small          */
#define RFA_ERR_HIP (-6)           /* a HIP runtime call failed               */

/* Library version (major*10000 + minor*100 + patch). */
int rfa_version(void);

/* Message describing the last error returned on this thread ("" if none). */
const char* rfa_last_error(void);

/* 1 if a causal / cross / decode kernel exists for feature width K and head dim d. */
int rfa_shape_supported(int K, int d);

/* Hardware self-check: runs one 16x16x32 fp16 MFMA tile product and one LDS
 * transposing read with known operands and compares with the lane layout the
 * kernels assume.  Returns RFA_OK when the layout matches. */
int rfa_selftest_layout(void* stream);

/* ---------------------------------------------------------------------------
 * Causal attention (training / prefill).
 *
 * rfa_causal_forward replaces rfa_cuda.forward(q, k, v)
 *   (random_feature_attention/cuda/rfa_cuda.cpp:22-27 -> RFAForward,
 *    cuda/forward.cu:128-169); formula: rfa.py:46-64.
 *   q, k : fp16 [T, N, K]   (time-major, as forward.cu:142-147 assumes)
 *   v    : fp16 [T, N, d]
 *   out  : fp16 [T, N, d]   every element is written
 * rfa_causal_backward replaces rfa_cuda.backward(q, k, v, grad_attn)
 *   (cuda/rfa_cuda.cpp:30-36 -> RFABackward, cuda/backward.cu:530-585);
 *   formula: rfa.py:66-103.
 *   grad_attn : fp16 [T, N, d];  dq, dk : fp16 [T, N, K];  dv : fp16 [T, N, d]
 * T = 0 or N = 0 is accepted and does nothing.
 * ------------------------------------------------------------------------- */
size_t rfa_causal_forward_workspace_bytes(int64_t T, int64_t N, int K, int d);
int rfa_causal_forward(const void* q, const void* k, const void* v, void* out, int64_t T,
                       int64_t N, int K, int d, void* workspace, size_t workspace_bytes,
                       void* stream);

size_t rfa_causal_backward_workspace_bytes(int64_t T, int64_t N, int K, int d);
int rfa_causal_backward(const void* q, const void* k, const void* v, const void* grad_attn,
                        void* dq, void* dk, void* dv, int64_t T, int64_t N, int K, int d,
                        void* workspace, size_t workspace_bytes, void* stream);

/* Number of time segments the causal kernels cut a sequence into for the given
 * shape (>= 1).  Environment variable RFA_HIP_NSEG overrides the heuristic. */
int rfa_causal_num_segments(int64_t T, int64_t N);

#ifdef __cplusplus
}
#endif
#endif /* RFA_HIP_H */
