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
 *     rfa_selftest_layout keeps its one result word in a static device variable;
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

/* Matrix-pipe rate probe for roofline figures: launches waves_per_simd (1..8) waves on every SIMD
 * of the device, each issuing iters x 8 independent 16x16x32 fp16 MFMAs on register operands (no
 * memory traffic), and stores the number of floating-point operations of the launch in *flops
 * (host memory).  The caller times the launch on its stream; sink is one float of device memory
 * that is never written in practice.  No counterpart in the reference. */
int rfa_selftest_mfma_rate(int waves_per_simd, int iters, float* sink, double* flops, void* stream);

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

/* rfa_causal_forward for callers that cannot allocate and have no workspace to pass (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): no counterpart in the
 * reference.  Same kernels and results as rfa_causal_forward; the segment totals live in a static
 * device array of rfa_static_scratch_bytes() = 16 MiB that every GPU the library runs on holds
 * until the process ends.  The call allocates and frees nothing.  Shapes whose
 * rfa_causal_forward_workspace_bytes exceed the array return RFA_ERR_WORKSPACE.  All calls on one
 * GPU share that GPU's array: calls that overlap in time on one GPU (two streams, two threads)
 * race; calls on one stream, one after the other, are fine (nothing in the array has to start
 * at zero: every total the scan reads is written earlier in the same call).  The first call on a
 * device looks the array's address up and sets kernel attributes: make it outside graph capture. */
size_t rfa_static_scratch_bytes(void);
int rfa_causal_forward_noalloc(const void* q, const void* k, const void* v, void* out, int64_t T,
                               int64_t N, int K, int d, void* stream);

/* Prefill for incremental decoding: rfa_causal_forward over a prompt of T steps that also
 * returns the state after the last step, s fp32 [N, K, d] and z fp32 [N, K] (every element
 * written; zero for T = 0), from which rfa_incremental / rfa_incremental_fused continue.
 * In the reference the same hand-off is T calls of incremental_rfa from a zero state
 * (causal_attention.py:17-54, saved_state keys "prev_s" / "prev_z" at :249-265).
 * Workspace: rfa_causal_forward_workspace_bytes. */
int rfa_causal_prefill(const void* q, const void* k, const void* v, void* out, float* s, float* z,
                       int64_t T, int64_t N, int K, int d, void* workspace, size_t workspace_bytes,
                       void* stream);

size_t rfa_causal_backward_workspace_bytes(int64_t T, int64_t N, int K, int d);
int rfa_causal_backward(const void* q, const void* k, const void* v, const void* grad_attn,
                        void* dq, void* dk, void* dv, int64_t T, int64_t N, int K, int d,
                        void* workspace, size_t workspace_bytes, void* stream);

/* Training-step variants (no counterpart in the reference, whose autograd Function
 * saves only q, k, v: rfa.py:124).  rfa_causal_forward_save additionally writes what
 * the backward pass can reuse into `saved` (rfa_causal_saved_state_bytes bytes, fp32: the
 * raw denominators and either the per-segment state totals or, where the backward runs as
 * one launch over state slices, the state after the last step); rfa_causal_backward_saved
 * reads them, and the forward output `out` (fp16 [T, N, d], as written by that forward
 * call), instead of recomputing the forward pass: with num = out * den the term
 * g . num of rfa.py:91 is (g . out) * den.  `saved` and `out` must come from a forward
 * call on the same q, k, v. */
size_t rfa_causal_saved_state_bytes(int64_t T, int64_t N, int K, int d);
int rfa_causal_forward_save(const void* q, const void* k, const void* v, void* out, void* saved,
                            size_t saved_bytes, int64_t T, int64_t N, int K, int d, void* workspace,
                            size_t workspace_bytes, void* stream);
int rfa_causal_backward_saved(const void* q, const void* k, const void* v, const void* grad_attn,
                              const void* out, const void* saved, size_t saved_bytes, void* dq, void* dk,
                              void* dv, int64_t T, int64_t N, int K, int d, void* workspace,
                              size_t workspace_bytes, void* stream);

/* A saved buffer describes itself: its first 256 bytes hold the plan of the forward call that
 * wrote it (16 ints: magic, version, layout, K, d, segments, steps per segment, scanned-totals
 * flag, T and N as two ints each, zeros), written on the device by that call.
 * rfa_causal_backward_saved runs with the plan recorded on the host when a forward call of this
 * process last wrote a buffer at that address (whatever the tuning knobs say by then), provided
 * that call had this call's T, N, K and d; for any other buffer (a copy, or an address the
 * caller's allocator has since given to another buffer) it assumes the current plan.  In every
 * case its kernels compare the header in the buffer with the plan they run, on the device: on a
 * mismatch dq, dk, dv are filled with NaN rather than computed from totals laid out
 * for another plan.  rfa_causal_backward_saved_workspace_bytes is the workspace that call needs
 * for a given saved buffer (= rfa_causal_backward_workspace_bytes unless the knobs changed since
 * the forward).  rfa_causal_saved_describe copies the 16 header ints to host memory and waits
 * for the stream (a debugging aid).  No counterpart in the reference. */
size_t rfa_causal_backward_saved_workspace_bytes(const void* saved, int64_t T, int64_t N, int K, int d);
int rfa_causal_saved_describe(const void* saved, int32_t* words16, void* stream);

/* Number of time segments the causal kernels cut a sequence into for the given
 * shape on the current device (>= 1). */
int rfa_causal_num_segments(int64_t T, int64_t N, int K, int d);

/* Launch-heuristic overrides for sweeps and tests (process-wide; -1 restores the heuristic):
 *   "nseg"  segments per sequence of the causal kernels (1..16)
 *   "prefix"  1/0: consumers read pre-scanned segment totals / add the totals up themselves
 *   "nseg_same"  1: the K = 256, d = 128 backward keeps the forward's segment length
 *   "free_wg"  workgroups the cross-attention readout and state backward aim for
 *   "project_streaming"  1: rfa_project_feature_map uses its streaming kernel for every shape
 *   "sliced"  1/0: rfa_causal_forward_save writes the final-state layout, whose backward is one
 *             launch that walks whole sequences by state slices (K <= 128; taken by itself at
 *             d = 64 when the slices cover 45 % of the compute units, at d = 128 only with K = 128
 *             and 90 %) / the
 *             segment-totals layout of the two-sweep backward
 *   "recompute"  1/0: the forward with K <= 128 runs as one launch without segment totals (every
 *             workgroup rebuilds the state at its segment's first step from the k, v rows before
 *             it; segments of unequal length) whenever no backward wants the totals / never.
 *             Unset: for up to 4 segments.  Its output has the bits of the one-segment scan.
 *   "prefix_cost"  cost of a rebuilt 64-step block in percent of a scanned one (default 12): moves
 *             the cut of that forward into segments
 *   "feature_wg"  workgroups the feature-map kernels aim for (default: one per compute unit for the
 *             eight-wave streaming kernels, 512 for the row-block backward of the wide shapes; in
 *             the backward each leaves one partial dW' for the reduction)
 * Initial values come from the environment variables RFA_HIP_<NAME>, read once per process and
 * never on the launch path.  No counterpart in the reference. */
int rfa_tuning_set(const char* name, int value);
int rfa_tuning_get(const char* name, int* value);

/* ---------------------------------------------------------------------------
 * Feature map  phi(x) = scale * [sin(W x^), cos(W x^)],  x^ = x / (||x|| + 1e-3).
 *
 * rfa_feature_map_forward replaces random_project(x=..., random_matrices=...)
 *   (random_feature_attention/utils.py:105-120, with _normalize :100-102); the
 *   reference fixes scale = SCALE = 0.1 (utils.py:10,119).
 *   x   : fp16 [R, H, d]   R = seq_len * bsz rows
 *   w   : fp16 [H, D, d]   the matrix build_random_matrices returns (utils.py:90-97)
 *   phi : fp16 [R, H, 2D]  sin block in columns [0, D), cos block in [D, 2D)
 * rfa_feature_map_backward is the gradient the reference obtains from autograd
 *   through those ATen calls: dx fp16 [R, H, d], dw fp32 [H, D, d] (summed over rows).
 * Supported: D in {32, 64, 128}, d in {64, 128} (rfa_feature_map_supported).
 * ------------------------------------------------------------------------- */
int rfa_feature_map_supported(int D, int d);

/* The matrix the feature map is taken with: W' = (sigma * W if sigma) / tau
 *   (build_random_matrices, random_feature_attention/utils.py:90-97; two elementwise ATen
 *   launches per call there, three more in the backward pass).  Same fp16 arithmetic: the
 *   product is rounded to fp16 before the division.
 *   w, out : fp16 [H, D, d];  sigma : fp16 [H, d] (the module's [H, 1, d] parameter,
 *   causal_attention.py:165) or NULL;  tau != 0.
 * rfa_build_random_matrices_backward: grad_out fp16 [H, D, d] -> dsigma fp16 [H, d] and/or
 *   dw fp16 [H, D, d] (either may be NULL), as autograd derives them from those launches. */
int rfa_build_random_matrices(const void* w, const void* sigma, float tau, void* out, int H, int D, int d,
                              void* stream);
int rfa_build_random_matrices_backward(const void* w, const void* sigma, const void* grad_out, float tau,
                                       void* dsigma, void* dw, int H, int D, int d, void* stream);
int rfa_feature_map_forward(const void* x, const void* w, void* phi, int64_t R, int H, int D, int d,
                            float scale, void* stream);
/* phi(x0) and phi(x1) through the same w in one launch: the q and k projections of a module
 * (causal_attention.py:241-248 calls random_project twice).  Same results as two
 * rfa_feature_map_forward calls. */
int rfa_feature_map_forward_pair(const void* x0, const void* x1, const void* w, void* phi0, void* phi1,
                                 int64_t R, int H, int D, int d, float scale, void* stream);
/* In the three backward entry points dw may be NULL: w then counts as a constant (random matrices
 * that are not reparametrised, utils.py:90-97 with reparam_proj off), only dx is formed, no
 * workspace is needed and the reduction launch is not made. */
size_t rfa_feature_map_backward_workspace_bytes(int64_t R, int H, int D, int d);
int rfa_feature_map_backward(const void* x, const void* w, const void* grad_phi, void* dx, float* dw,
                             int64_t R, int H, int D, int d, float scale, void* workspace,
                             size_t workspace_bytes, void* stream);
/* Two tensors that went through the same w (phi(q) and phi(k) of a module, causal_attention.py:246-247)
 *   differentiated in one launch: dx0, dx1 as above, dw = the sum of both contributions (what
 *   autograd accumulates into w there). */
size_t rfa_feature_map_backward_pair_workspace_bytes(int64_t R, int H, int D, int d);
int rfa_feature_map_backward_pair(const void* x0, const void* x1, const void* w, const void* grad_phi0,
                                  const void* grad_phi1, void* dx0, void* dx1, float* dw, int64_t R, int H,
                                  int D, int d, float scale, void* workspace, size_t workspace_bytes,
                                  void* stream);

/* The same launch for the backward of a module's three input projections
 * (causal_attention.py:228-247 under autograd, where the gradients of q_proj's, k_proj's and
 * v_proj's outputs each meet their weight in a GEMM of their own): with E = H * d, `packed` is
 * fp16 [R, 3E] and receives  [ dx0 | dx1 | third ]  side by side -- dx0, dx1 as above, `third` (fp16
 * [R, E], e.g. the gradient of v; may be NULL: that block is left untouched) copied by further
 * workgroups of the launch -- so that one product  packed x [Wq; Wk; Wv]  gives the gradient of the
 * projections' input and one  packed^T x  all three weight gradients.  dw and the workspace as for
 * rfa_feature_map_backward_pair. */
int rfa_feature_map_backward_pair_packed(const void* x0, const void* x1, const void* w, const void* grad_phi0,
                                         const void* grad_phi1, const void* third, void* packed, float* dw,
                                         int64_t R, int H, int D, int d, float scale, void* workspace,
                                         size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Linear projections to heads with the feature map in the epilogue.
 *
 * rfa_project_feature_map replaces, in one launch, the chain the attention modules run on
 * their input: q_proj / k_proj / v_proj (torch.nn.Linear), the view to heads and
 * random_project on the q and k projections
 *   (random_feature_attention/causal_attention.py:228-247; cross_attention.py:66-76 for the
 *    k / v projections of the encoder output, :279-283 for the q projection; utils.py:100-120).
 *   x        : fp16 [R, E]      R = seq_len * bsz rows, E a multiple of 64
 *   weights  : np pointers (1 <= np <= 3) to fp16 [H*d, E], torch.nn.Linear.weight layout
 *   biases   : np pointers to fp16 [H*d] (8-byte aligned); the array or any entry may be NULL
 *   y        : np pointers to fp16 [R, H, d]   y_p = x W_p^T + b_p (the backward of the feature
 *              map needs it); an entry may be NULL where phi[p] is not: that projection then
 *              leaves only phi(y_p) behind (inference, no backward pass)
 *   phi      : np pointers to fp16 [R, H, 2D], or NULL entries (or a NULL array): projection p
 *              gets phi(y_p) only where phi[p] is non-NULL
 *   w_feat   : fp16 [H, D, d] as for rfa_feature_map_forward; may be NULL if no phi is asked for
 * The pointer arrays themselves live in host memory and are read during the call only.
 * With every phi NULL this is a plain batched Linear (e.g. out_proj,
 * causal_attention.py:278) and D only has to be a supported value.
 * ------------------------------------------------------------------------- */
int rfa_project_feature_map(const void* x, const void* const* weights, const void* const* biases,
                            void* const* y, void* const* phi, int np, const void* w_feat, int64_t R,
                            int E, int H, int D, int d, float scale, void* stream);

/* rfa_linear_weight_grad: weight and bias gradients of those Linear layers, what autograd
 * computes for torch.nn.Linear in the backward of the lines cited above,
 *     dW_p [E_out, E_in] = dy_p^T x,    db_p [E_out] = column sums of dy_p,
 * for np (1..3) layers that share the input x, as a row-split MFMA contraction plus a reduction.
 *   x  : fp16 [R, E_in]      dy : np pointers to fp16 [R, E_out]
 *   dw : np pointers to fp16 [E_out, E_in]      db : np pointers to fp16 [E_out] or NULL entries
 *        (or a NULL array)
 *   E_out, E_in multiples of 128; workspace of rfa_linear_weight_grad_workspace_bytes bytes. */
size_t rfa_linear_weight_grad_workspace_bytes(int64_t R, int E_out, int E_in, int np);
int rfa_linear_weight_grad(const void* x, const void* const* dy, void* const* dw, void* const* db, int np,
                           int64_t R, int E_out, int E_in, void* workspace, size_t workspace_bytes,
                           void* stream);

/* ---------------------------------------------------------------------------
 * Cross attention (encoder -> decoder).  The state is fp32.
 *
 * rfa_cross_state replaces the two reductions of
 *   CrossAttentionProjectLayer.project_and_reshape
 *   (random_feature_attention/cross_attention.py:97-104):
 *     s[b,h] = sum_s phi_k[s,b,h] (x) v[s,b,h] ;  z[b,h] = sum_s phi_k[s,b,h]
 *   phi_k : fp16 [S, B*H, K];  v : fp16 [S, B*H, d]
 *   key_padding_mask : bytes [B, S], non-zero = padded key (its phi_k row counts
 *                      as zero, cross_attention.py:97-100), or NULL
 *   s : fp32 [B*H, K, d];  z : fp32 [B*H, K]     (overwritten)
 * rfa_cross_readout replaces CrossAttention.rfa after the feature map
 *   (cross_attention.py:266-269):  out = (phi_q s) / max(|phi_q z|, 1)
 *   phi_q : fp16 [T, N, K];  out : fp16 [T, N, d]
 * The two *_backward functions are the gradients the reference obtains from
 * autograd through those einsums:
 *   readout: dphi_q fp16 [T, N, K], ds fp32 [N, K, d], dz fp32 [N, K] (overwritten)
 *   state  : dphi_k fp16 [S, N, K] (zero rows at padded keys), dv fp16 [S, N, d]
 * ------------------------------------------------------------------------- */
int rfa_cross_state(const void* phi_k, const void* v, const uint8_t* key_padding_mask, float* s, float* z,
                    int64_t S_len, int64_t B, int H, int K, int d, void* stream);
int rfa_cross_readout(const void* phi_q, const float* s, const float* z, void* out, int64_t T, int64_t N,
                      int K, int d, void* stream);
int rfa_cross_readout_backward(const void* phi_q, const float* s, const float* z, const void* grad_attn,
                               void* dphi_q, float* ds, float* dz, int64_t T, int64_t N, int K, int d,
                               void* stream);
int rfa_cross_state_backward(const void* phi_k, const void* v, const uint8_t* key_padding_mask,
                             const float* ds, const float* dz, void* dphi_k, void* dv, int64_t S_len,
                             int64_t B, int H, int K, int d, void* stream);

/* ---------------------------------------------------------------------------
 * Quadratic form with explicit masks: masked_rfa(phi_q, phi_k, v, key_padding_mask,
 * attn_mask) (random_feature_attention/causal_attention.py:57-109), the path
 * CausalAttention takes with cuda_causal_rfa = False, and its gradient (autograd of
 * the same lines).  Weights a[t][s] = phi_q[t] . phi_k[s], zero where key s is padded
 * or attn_mask[t][s] is set, divided by max(|row sum|, 1e-3) (utils.py:123-130),
 * applied to v.
 *   phi_q, phi_k : fp16 [T, N, K]  (N = B * H, time-major);  v, out, grad_attn : fp16 [T, N, d]
 *   key_padding_mask : bytes [B, T], non-zero = padded key, may be NULL
 *   attn_mask        : bytes [T, Tp], non-zero = masked (the reference's `attn_mask < 0`),
 *                      Tp = T rounded up to a multiple of 64, padding columns non-zero; may be NULL
 *   attn_mask_t      : its transpose, bytes [T (key), Tp (query)], padded the same way
 *   rsum             : fp32 [T, N] raw row sums (forward: optional output; backward: input)
 *   dphi_q, dphi_k, dv : every element written; a padded key gets zero dphi_k and dv.
 * ------------------------------------------------------------------------- */
int rfa_masked_forward(const void* phi_q, const void* phi_k, const void* v, const uint8_t* key_padding_mask,
                       const uint8_t* attn_mask, void* out, float* rsum, int64_t T, int64_t Tp, int64_t B,
                       int H, int K, int d, void* stream);
size_t rfa_masked_backward_workspace_bytes(int64_t T, int64_t N, int d);
int rfa_masked_backward(const void* phi_q, const void* phi_k, const void* v, const void* grad_attn,
                        const void* out, const float* rsum, const uint8_t* key_padding_mask,
                        const uint8_t* attn_mask, const uint8_t* attn_mask_t, void* dphi_q, void* dphi_k,
                        void* dv, int64_t T, int64_t Tp, int64_t B, int H, int K, int d, void* workspace,
                        size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Incremental decoding.  The fp32 state (s [N, K, d], z [N, K]) is updated IN
 * PLACE; one kernel is launched per step, in order, on `stream`.
 *
 * rfa_incremental replaces incremental_rfa(phi_q=, phi_k=, v=, s=, z=)
 *   (random_feature_attention/causal_attention.py:17-54), whose loop over tgt_len
 *   is the `steps` loop here:
 *   phi_q, phi_k : fp16 [steps, N, K];  v : fp16 [steps, N, d];  out : fp16 [steps, N, d]
 * rfa_incremental_fused additionally evaluates the feature map of the raw projected
 *   q, k inside the step kernel, i.e. the decode branch of CausalAttention.forward
 *   (causal_attention.py:241-265) in one launch per token:
 *   q, k, v : fp16 [steps, B, H, d];  w : fp16 [H, D, d];  K = 2D
 * ------------------------------------------------------------------------- */
int rfa_incremental(const void* phi_q, const void* phi_k, const void* v, float* s, float* z, void* out,
                    int64_t steps, int64_t N, int K, int d, void* stream);
int rfa_incremental_fused(const void* q, const void* k, const void* v, const void* w, float scale, float* s,
                          float* z, void* out, int64_t steps, int64_t B, int H, int D, int d, void* stream);
/* The same steps with the state read from s_in, z_in and the advanced state written to s_out,
 * z_out (the first step reads the inputs, later steps advance the outputs in place), as the
 * reference's `s = s + ...` leaves the caller's tensors alone (causal_attention.py:42-43).
 * Same traffic as the in-place form; s_out, z_out may alias s_in, z_in. */
int rfa_incremental_out(const void* phi_q, const void* phi_k, const void* v, const float* s_in, const float* z_in,
                        float* s_out, float* z_out, void* out, int64_t steps, int64_t N, int K, int d,
                        void* stream);
int rfa_incremental_fused_out(const void* q, const void* k, const void* v, const void* w, float scale,
                              const float* s_in, const float* z_in, float* s_out, float* z_out, void* out,
                              int64_t steps, int64_t B, int H, int D, int d, void* stream);
/* The same step for callers whose q, k and v come out of ONE projection (a Linear layer whose
 * weight stacks q_proj, k_proj, v_proj of causal_attention.py:228-247: one small-M GEMM per token
 * instead of three): qkv fp16 [steps, B, 3, H, d], i.e. rows of 3 * H * d with q, k, v in their
 * thirds.  State read from s_in, z_in and written to s_out, z_out, which may be the same
 * buffers (in place).  Same results as rfa_incremental_fused(_out) on the three thirds. */
int rfa_incremental_qkv(const void* qkv, const void* w, float scale, const float* s_in, const float* z_in,
                        float* s_out, float* z_out, void* out, int64_t steps, int64_t B, int H, int D, int d,
                        void* stream);

/* ---------------------------------------------------------------------------
 * Per-kernel timing (no counterpart in the reference; used by bench.py).
 * While enabled, every kernel launch of this library is bracketed by a HIP event
 * pair on its stream.  rfa_profile_collect waits for the recorded pairs and adds
 * their elapsed times to per-kernel totals; rfa_profile_get reads one total
 * (index in [0, rfa_profile_kernel_count())); rfa_profile_reset clears them.
 * ------------------------------------------------------------------------- */
int rfa_profile_enable(int on);
int rfa_profile_collect(void);
int rfa_profile_reset(void);
int rfa_profile_kernel_count(void);
int rfa_profile_get(int index, const char** name, double* total_ms, int64_t* calls);

#ifdef __cplusplus
}
#endif
#endif /* RFA_HIP_H */
