/*
 * cottention.h -- C ABI of libcottention_hip.so: cosine linear attention for AMD MI355X (gfx950).
 *
 * This is the boundary a host binds instead of the reference's pybind/ATen extension.  All entry
 * points take raw device pointers, plain sizes and a HIP stream (passed as void*; NULL = the
 * default stream).  The library never allocates, frees or synchronises: outputs and workspaces
 * are caller-owned device memory, kernels are enqueued on the given stream and the call returns.
 *
 * Tensors are contiguous row-major (B, H, N, D) exactly as the reference kernels index them
 * (Cuda_Kernel/combined_kernel_general.cu:136 `((n*H+h)*S+s)*D+d`).  Pointers must be 16-byte
 * aligned.  `dtype` selects the storage type of q/k/v/o; accumulation is fp32 (fp64 for
 * COTT_F64), unlike the reference, which accumulates in the storage type (:121,:133).
 *
 * Every function returns COTT_OK or an error code; cott_last_error() gives the text for the most
 * recent failure on the calling thread.  Shape rules follow combined_kernel_general.cu:365-374:
 * q and k share their last dimension, every head dimension is a multiple of 16 and at least 32.
 */
#ifndef COTTENTION_H
#define COTTENTION_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define COTT_API __attribute__((visibility("default")))

#define COTT_OK 0
#define COTT_ERR_INVALID 1     /* bad pointer, shape or flag                        */
#define COTT_ERR_UNSUPPORTED 2 /* legal request this build has no kernel for       */
#define COTT_ERR_WORKSPACE 3   /* workspace missing or smaller than required       */
#define COTT_ERR_HIP 4         /* the HIP runtime reported a launch error          */

typedef enum cott_dtype {
    COTT_F32 = 0,  /* kernel.float32  : combined_kernel_general.cu:445 */
    COTT_F64 = 1,  /* kernel.float64  : :446                           */
    COTT_F16 = 2,  /* kernel.float16  : :447                           */
    COTT_BF16 = 3  /* kernel.bfloat16 : :449                           */
} cott_dtype;

/* Library version, major*10000 + minor*100 + patch. */
COTT_API int cott_version(void);

/* Text of the last error raised on this thread ("" if none).  Replaces the c10::Error that
 * TORCH_CHECK throws in combined_kernel_general.cu:355-374. */
COTT_API const char *cott_last_error(void);

/* ---- generic causal op ---------------------------------------------------------------------
 *   o[s,j] = sum_i q[s,i] * sum_{s' <= s (>= s if reversed)} k[s',i] * v[s',j]
 * Replaces kernel_call<T> / forward_<T>, Cuda_Kernel/combined_kernel_general.cu:257-289,352-429
 * (Python: FastAttention2.kernel.<dtype>(Q,K,V,block_size,inplace,reversed), :444-454).
 * q,k: (B,H,N,Dk); v,o: (B,H,N,Dv).  The diagonal s'=s is included.  `reversed` is the flag of
 * :126-130.  Workspace: cott_causal_workspace_bytes() bytes of device memory (may be 0). */
COTT_API size_t cott_causal_workspace_bytes(int B, int H, int N, int Dk, int Dv, int dtype);
COTT_API int cott_causal_fwd(const void *q, const void *k, const void *v, void *o,
                    int B, int H, int N, int Dk, int Dv, int dtype, int reversed,
                    void *workspace, size_t workspace_bytes, void *stream);
/* inplace=True of forward_<T> (combined_kernel_general.cu:403-404: the output tensor IS V).  Returns 1 when
 * cott_causal_fwd may be called with o == v for this shape and dtype (every workgroup has read the rows and
 * columns of v it needs before it, or any other workgroup, writes them as o): the MFMA kernels, i.e. bf16 / fp16 /
 * fp32 with head dims 32..128 in steps of 16.  0: the caller computes into a temporary and copies.  Only the exact
 * alias o == v is covered; q and k must not overlap o. */
COTT_API int cott_causal_fwd_may_alias_v(int B, int H, int N, int Dk, int Dv, int dtype);

/* ---- causal forward that takes no workspace and allocates nothing ------------------------------
 * cott_causal_fwd with the group-state slots (its workspace) kept in a device array built into the library
 * instead of caller memory.  It has no counterpart in the reference; it is for callers that cannot allocate
 * device memory around the call: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  Same arguments, results (bit for bit) and errors as cott_causal_fwd; a shape whose slots exceed
 * cott_noalloc_scratch_bytes() (48 MiB, enough for every plan this build makes on a part of up to 256 CUs)
 * returns COTT_ERR_WORKSPACE.
 * The array's address is looked up once per device (hipGetSymbolAddress): by cott_noalloc_scratch_bytes() when a
 * device is current, else by the first call of the entry point on that device.  Call cott_noalloc_scratch_bytes()
 * before a stream capture starts, so that the lookup does not happen inside it.  No call allocates or frees.
 * All calls on one GPU share that GPU's array: calls that may overlap on one GPU (different streams or threads)
 * race on it and must be ordered by the caller.  Keep cott_profile_enable off (it creates HIP events). */
COTT_API size_t cott_noalloc_scratch_bytes(void);
COTT_API int cott_causal_fwd_noalloc(const void *q, const void *k, const void *v, void *o,
                            int B, int H, int N, int Dk, int Dv, int dtype, int reversed, void *stream);

/* ---- causal forward with state hand-over (prefill -> decode, or a sequence fed in pieces) -----
 *   o[s,j] = sum_i q[s,i] * ( state_in[i,j] + sum_{s' <= s} k[s',i] * v[s',j] )
 *   state_out[i,j] = state_in[i,j] + sum_{s' < N} k[s',i] * v[s',j]
 * Replaces the per-token Python loop that the reference runs over a prompt to build its decode
 * state (GPT_Trainer/GPTCosAttention.py:253-272; generation driver fast_infer.py:111): one call
 * over the prompt yields the outputs of cott_causal_fwd AND the state that cott_decode_step
 * continues from.  state_in / state_out: (B,H,Dk,Dv) fp32 (fp64 for COTT_F64), the layout of
 * cott_decode_step; either may be NULL (start from zero / state not wanted); they may alias.
 * Workspace: cott_causal_workspace_bytes().  N == 0 copies state_in to state_out. */
COTT_API int cott_causal_fwd_state(const void *q, const void *k, const void *v, void *o,
                          const void *state_in, void *state_out,
                          int B, int H, int N, int Dk, int Dv, int dtype,
                          void *workspace, size_t workspace_bytes, void *stream);

/* ---- causal backward ------------------------------------------------------------------------
 * (dq, dk, dv) of o = cott_causal_fwd(q,k,v) contracted with d_o.  Replaces the three launches
 * of CustomAttention.backward, Cuda_Kernel/Custom_Kernel.py:106-108 (closed forms :63,:68,:72)
 * and the older fused entry point backward_<T>, Cuda_Kernel/backwardv2_comb.cu:172-224
 * (Python: FastAttention.backward.<dtype>(Q,K,V,prev_grad,block_size) -> [dQ,dK,dV]).
 * d_o, dv: (B,H,N,Dv); dq, dk: (B,H,N,Dk). */
COTT_API size_t cott_causal_bwd_workspace_bytes(int B, int H, int N, int Dk, int Dv, int dtype);
COTT_API int cott_causal_bwd(const void *q, const void *k, const void *v, const void *d_o,
                    void *dq, void *dk, void *dv,
                    int B, int H, int N, int Dk, int Dv, int dtype,
                    void *workspace, size_t workspace_bytes, void *stream);

/* ---- causal forward / backward with states saved for the backward pass -----------------------
 * dq sums over the past, dk and dv over the future.  Started from the sum of k^T v over the whole sequence (or, when
 * heads are cut into sequence groups, over everything before a group's end) dq can be computed walking the sequence
 * from its end like the other two, so that the three read the same rows of q, k, v and d_o at the same time and the
 * gradient launch fetches each tensor once instead of nearly twice.  cott_causal_bwd has to get those sums from an
 * extra pass over k and v (and only does for heads cut into groups); the forward pass carries exactly these states,
 * so a training step can have them written there (16 KiB per head at the headline shape, a few MiB on long
 * sequences): what CustomAttention.forward saves for backward (Cuda_Kernel/Custom_Kernel.py:16,
 * ctx.save_for_backward) grows by one small tensor.
 *   cott_causal_saved_plan   chunks_per_cut, ncuts (0 = this shape's backward pass takes no saved states: use the
 *                            plain entry points), the floats per saved slot and the workspace
 *                            cott_causal_bwd_saved needs.  Plans exist for sequences of 16 chunks or more whose
 *                            gradients run as dq beside a (dk, dv) pair of workgroups (square head dims up to 64)
 *                            or as three problems cut into sequence groups.
 *   cott_causal_fwd_save     cott_causal_fwd (not reversed; same o, bit for bit) that also writes
 *                            saved: (B,H,ncuts,slot_floats) fp32, slot g = sum over the positions before
 *                            64 * (ceil(N/64) - g * chunks_per_cut) of k^T v  (slot 0: the whole sequence).
 *                            Workspace: cott_causal_workspace_bytes().
 *   cott_causal_bwd_saved    cott_causal_bwd with dq seeded from `saved` (same results to rounding).
 * A slot holds the (Dk,Dv) state padded to (P(Dk),P(Dv)), P(d) = 32, 64 or 128, as 16 x 16 tiles in the MFMA
 * accumulator layout, so that the forward pass writes it with one 16-byte store per lane and tile: element
 * [16 it + 4 g + c][16 jt + m] is float ((it * P(Dv)/16 + jt) * 64 + 16 g + m) * 4 + c of the slot; tiles outside
 * (Dk,Dv) are not written.  The array only has a meaning for the shape and dtype it was made for.
 * bf16 / fp16, head dims 32..128 in steps of 16; other cases return COTT_ERR_UNSUPPORTED. */
COTT_API int cott_causal_saved_plan(int B, int H, int N, int Dk, int Dv, int dtype,
                           int *chunks_per_cut, int *ncuts, int *slot_floats, size_t *bwd_workspace_bytes);
COTT_API int cott_causal_fwd_save(const void *q, const void *k, const void *v, void *o,
                         float *saved, int chunks_per_cut, int ncuts,
                         int B, int H, int N, int Dk, int Dv, int dtype,
                         void *workspace, size_t workspace_bytes, void *stream);
COTT_API int cott_causal_bwd_saved(const void *q, const void *k, const void *v, const void *d_o,
                          void *dq, void *dk, void *dv,
                          const float *saved, int chunks_per_cut, int ncuts,
                          int B, int H, int N, int Dk, int Dv, int dtype,
                          void *workspace, size_t workspace_bytes, void *stream);
/* The same pair with o (forward) / d_o (backward) laid out (B,N,H,Dv), as cott_causal_fwd_bnhd / cott_causal_bwd_bnhd
 * (the head merge of GPT_Trainer/GPTCosAttention.py:106-113 without its copy); `saved` is the same array. */
COTT_API int cott_causal_fwd_save_bnhd(const void *q, const void *k, const void *v, void *o,
                              float *saved, int chunks_per_cut, int ncuts,
                              int B, int H, int N, int Dk, int Dv, int dtype,
                              void *workspace, size_t workspace_bytes, void *stream);
COTT_API int cott_causal_bwd_saved_bnhd(const void *q, const void *k, const void *v, const void *d_o,
                               void *dq, void *dk, void *dv,
                               const float *saved, int chunks_per_cut, int ncuts,
                               int B, int H, int N, int Dk, int Dv, int dtype,
                               void *workspace, size_t workspace_bytes, void *stream);

/* ---- causal forward / backward with the head merge folded in --------------------------------
 * The same two operations with the attention output o (forward) and its gradient d_o (backward) laid out
 * (B,N,H,Dv), i.e. as the rows of the (B,N,H*Dv) tensor that the output projection reads and
 * differentiates.  Replaces the permute + contiguous copy of the head merge around the op
 * (GPT_Trainer/GPTCosAttention.py:106-113 `_merge_heads`, called at :500, and its backward).  q, k, v and
 * dq, dk, dv stay (B,H,N,D) (cott_prep_ex_* already reads and writes the projection layout on that side).
 * bf16 / fp16, head dims 32..128 in steps of 16, N*H*D <= 2^30; other cases return COTT_ERR_UNSUPPORTED
 * and the caller permutes.  Workspace: cott_causal_workspace_bytes / cott_causal_bwd_workspace_bytes. */
COTT_API int cott_causal_fwd_bnhd(const void *q, const void *k, const void *v, void *o,
                         int B, int H, int N, int Dk, int Dv, int dtype,
                         void *workspace, size_t workspace_bytes, void *stream);
COTT_API int cott_causal_bwd_bnhd(const void *q, const void *k, const void *v, const void *d_o,
                         void *dq, void *dk, void *dv,
                         int B, int H, int N, int Dk, int Dv, int dtype,
                         void *workspace, size_t workspace_bytes, void *stream);

/* ---- non-causal form ------------------------------------------------------------------------
 *   o = q (k^T v)   per (batch, head)
 * Replaces the two einsums of BERT_Trainer/BertCosAttention.py:249 (the (QK^T)V branch at :222
 * is the same value).  Backward: dq = d_o (v^T k), dk = v (d_o^T q)
 * (GPT_Trainer/GPTCosAttention.py:34-35), dv = k (q^T d_o). */
COTT_API size_t cott_noncausal_workspace_bytes(int B, int H, int N, int Dk, int Dv, int dtype);
COTT_API int cott_noncausal_fwd(const void *q, const void *k, const void *v, void *o,
                       int B, int H, int N, int Dk, int Dv, int dtype,
                       void *workspace, size_t workspace_bytes, void *stream);
COTT_API int cott_noncausal_bwd(const void *q, const void *k, const void *v, const void *d_o,
                       void *dq, void *dk, void *dv,
                       int B, int H, int N, int Dk, int Dv, int dtype,
                       void *workspace, size_t workspace_bytes, void *stream);

/* Non-causal form with o / d_o laid out (B,N,H,Dv): the context-layer permute of
 * BERT_Trainer/BertCosAttention.py:317 and its backward without the copy.  Same limits as
 * cott_causal_fwd_bnhd; workspace: cott_noncausal_workspace_bytes. */
COTT_API int cott_noncausal_fwd_bnhd(const void *q, const void *k, const void *v, void *o,
                            int B, int H, int N, int Dk, int Dv, int dtype,
                            void *workspace, size_t workspace_bytes, void *stream);
COTT_API int cott_noncausal_bwd_bnhd(const void *q, const void *k, const void *v, const void *d_o,
                            void *dq, void *dk, void *dv,
                            int B, int H, int N, int Dk, int Dv, int dtype,
                            void *workspace, size_t workspace_bytes, void *stream);

/* ---- recurrent decode step ------------------------------------------------------------------
 *   S[b,h,dk,dv] += k[b,h,dk] * v[b,h,dv] ;  o[b,h,dv] = sum_dk q[b,h,dk] * S[b,h,dk,dv]
 * Replaces the per-token body of GPT_Trainer/GPTCosAttention.py:262-269 (:264 update, :267 read;
 * the output uses the UPDATED state).  `state` is caller-owned, (B,H,Dk,Dv), fp32 (fp64 for
 * COTT_F64) and updated in place; the reference keeps the transposed orientation (B,H,Dv,Dk) in
 * fp64 (:80).  q,k: (B,H,Dk); v,o: (B,H,Dv) in `dtype`.  Needs no workspace. */
COTT_API int cott_decode_step(void *state, const void *q, const void *k, const void *v, void *o,
                     int B, int H, int Dk, int Dv, int dtype, void *stream);

/* The same step on the RAW projections of the new token: the GPT-J rotation of the first rotary_dim columns of q
 * and k by row `position` of rot_table ((table_rows, rotary_dim) fp32, [sin | cos]; NULL = no rotation; the row is
 * clamped to the table), the L2 normalisation of q and k and v / max(cnt^sig[h], 1) (sig: (H) fp32 =
 * sigmoid(norm_const), NULL = no scaling; cnt = tokens so far including this one) run inside the kernel: one
 * launch per token and layer instead of the separate elementwise kernels of
 * GPT_Trainer/GPTCosAttention.py:229-248,462-476 in front of :264-267.  q, k: (B,H,Dk) = the (B,1,H,Dk)
 * projection output; Dv in {32,64,128,256}, Dk <= 256. */
COTT_API int cott_decode_step_prep(void *state, const void *q, const void *k, const void *v, void *o,
                          const float *sig, float cnt, const float *rot_table, long long position,
                          int rotary_dim, int table_rows,
                          int B, int H, int Dk, int Dv, int dtype, void *stream);

/* ---- fused input preparation (the elementwise work the module does before the attention op) --
 *   q_out = keep * q / max(|q|_2, 1e-12)     (rows of Dk; same for k)
 *   v_out = keep * v / max(cnt^sig[h], 1)    (rows of Dv)
 * in one pass per tensor, converting in_dtype -> out_dtype on the way.  Replaces the eight
 * elementwise / reduction kernels of GPT_Trainer/GPTCosAttention.py:229-248 (normalize :229-230,
 * value scaling :234-241, mask multiplies :243-248) and BERT_Trainer/BertCosAttention.py:162-178
 * (for a 0/1 mask the order mask/normalise/scale does not matter).
 * keep: (B,N) bytes, 0 = padded position, or NULL.  cnt: (B,N) fp32, the number of kept keys a
 * position attends to (GPT: running count, :228; BERT: the total, :178) and sig: (H) fp32 =
 * sigmoid(norm_const); both NULL = no value scaling.  fp64 converts only to fp64.
 * cott_prep_bwd: gq,gk,gv = gradients wrt the outputs (grad_dtype); dq,dk,dv = gradients wrt the
 * inputs (in_dtype); dsig_rows (B,H,N) fp32 or NULL receives per-row d/dsig[h] (sum it over B,N). */
COTT_API int cott_prep_fwd(const void *q, const void *k, const void *v, void *q_out, void *k_out, void *v_out,
                  const unsigned char *keep, const float *cnt, const float *sig,
                  int B, int H, int N, int Dk, int Dv, int in_dtype, int out_dtype, void *stream);
COTT_API int cott_prep_bwd(const void *q, const void *k, const void *v,
                  const void *gq, const void *gk, const void *gv, void *dq, void *dk, void *dv,
                  float *dsig_rows, const unsigned char *keep, const float *cnt, const float *sig,
                  int B, int H, int N, int Dk, int Dv, int in_dtype, int grad_dtype, void *stream);

/* The same with the two steps that surround it in the GPT block folded in (GPTCosAttention.py:444-479):
 * in_bnhd != 0: q, k, v (and, backward, dq, dk, dv) are laid out (B,N,H,D), as the projections produce them
 * (the outputs / incoming gradients stay (B,H,N,D)), which removes the permute + contiguous copies of :478-479 and
 * Custom_Kernel.py:11-13;  rot_table != NULL: the GPT-J rotary embedding (apply_rotary_pos_emb, :462-476) is
 * applied to the first rotary_dim columns of q and k before normalisation.  rot_table: (table_rows, rotary_dim)
 * fp32, row p = [sin(p f_i) | cos(p f_i)]; pos: (B,N) int64 row index per position; an index outside [0, table_rows) is clamped
 * to the table on the device, nothing reports it. */
COTT_API int cott_prep_ex_fwd(const void *q, const void *k, const void *v, void *q_out, void *k_out, void *v_out,
                     const unsigned char *keep, const float *cnt, const float *sig,
                     const float *rot_table, const long long *pos, int rotary_dim, int table_rows, int in_bnhd,
                     int B, int H, int N, int Dk, int Dv, int in_dtype, int out_dtype, void *stream);
COTT_API int cott_prep_ex_bwd(const void *q, const void *k, const void *v,
                     const void *gq, const void *gk, const void *gv, void *dq, void *dk, void *dv,
                     float *dsig_rows, const unsigned char *keep, const float *cnt, const float *sig,
                     const float *rot_table, const long long *pos, int rotary_dim, int table_rows, int in_bnhd,
                     int B, int H, int N, int Dk, int Dv, int in_dtype, int grad_dtype, void *stream);

/* ---- causal forward on the RAW projections: the input preparation inside the attention kernel ------------
 *   o = cott_causal_fwd(q_hat, k_hat, v_hat)  with
 *   q_hat = keep * rot(q) / max(|rot(q)|, 1e-12),  k_hat likewise,  v_hat = keep * v / max(cnt^sig[h], 1)
 * in ONE launch: the rows are rotated, normalised, scaled and masked on their way into the kernel's tiles, so the
 * separate pass of cott_prep_ex_fwd (one read and one write of q, k, v) disappears from the forward of the block
 * (GPT_Trainer/GPTCosAttention.py:229-248 normalise / scale / mask and :462-476 rotary, in front of :282).
 * q_out, k_out, v_out: (B,H,N,D) receive q_hat, k_hat, v_hat for the backward pass (cott_causal_bwd on them, then
 * cott_prep_ex_bwd); any of them may be NULL.  keep, cnt, sig as in cott_prep_fwd.  rot_table: (table_rows,
 * rotary_dim) fp32 as in cott_prep_ex_fwd, rotary_dim a multiple of 8, or NULL; the table row of position s of batch
 * element b is pos_ids[b * N + s] (position_ids of GPT_Trainer/GPTCosAttention.py:458: int64, (B,N), any values) or,
 * with pos_ids NULL, pos0 + s; rows outside the table are clamped to it.  in_bnhd: q, k, v
 * are (B,N,H,D); o_bnhd: o is (B,N,H,Dv).  bf16 / fp16; head dims 32..128 in steps of 16 (with Dk above 64 the value
 * tiles must be 64 or 128 columns wide after any split into column halves, i.e. Dv above 32 resp. 64):
 * cott_causal_fwd_prep_supported() says (1 / 0) whether a shape qualifies; otherwise the call returns
 * COTT_ERR_UNSUPPORTED and the caller prepares the inputs with cott_prep_ex_fwd.  workspace: as cott_causal_fwd for the
 * same shape (cott_causal_workspace_bytes; sequences cut into groups, whose group sums are then formed from rows
 * prepared the same way; NULL / 0 when that is 0). */
COTT_API int cott_causal_fwd_prep_supported(int B, int H, int N, int Dk, int Dv, int dtype, int rotary_dim);
/* 1 where the one launch has also measured faster than cott_prep_ex_fwd followed by cott_causal_fwd (every shape but
 * those planned as column halves in sequence groups: few heads, medium sequence lengths), else 0: the rule the
 * modules of this package follow when they choose between the two forms.  Pure host function. */
COTT_API int cott_causal_fwd_prep_preferred(int B, int H, int N, int Dk, int Dv, int dtype, int rotary_dim);
COTT_API int cott_causal_fwd_prep(const void *q, const void *k, const void *v, void *o,
                         void *q_out, void *k_out, void *v_out,
                         const unsigned char *keep, const float *cnt, const float *sig,
                         const float *rot_table, const long long *pos_ids, long long pos0, int rotary_dim, int table_rows,
                         int in_bnhd, int o_bnhd,
                         int B, int H, int N, int Dk, int Dv, int dtype,
                         void *workspace, size_t workspace_bytes, void *stream);
/* The non-causal counterpart: o = q_hat (k_hat^T v_hat) on the raw projections in one launch, q_hat, k_hat, v_hat as
 * above without a rotation (BERT_Trainer/BertCosAttention.py:162-178 mask / normalise / scale in front of :249; there
 * cnt is the number of real tokens of the batch element at every position).  q_out, k_out, v_out receive the
 * prepared tensors for the backward pass (cott_noncausal_bwd on them, then cott_prep_ex_bwd).  bf16 / fp16, head
 * dims 32..128 in steps of 16, and a head must fit one workgroup (no sequence groups: B*H at least about the number
 * of CUs): cott_noncausal_fwd_prep_supported() says whether a shape qualifies; otherwise COTT_ERR_UNSUPPORTED.
 * Needs no workspace. */
COTT_API int cott_noncausal_fwd_prep_supported(int B, int H, int N, int Dk, int Dv, int dtype);
COTT_API int cott_noncausal_fwd_prep(const void *q, const void *k, const void *v, void *o,
                            void *q_out, void *k_out, void *v_out,
                            const unsigned char *keep, const float *cnt, const float *sig,
                            int in_bnhd, int o_bnhd,
                            int B, int H, int N, int Dk, int Dv, int dtype, void *stream);
/* ... that also writes the states the backward pass takes (cott_causal_saved_plan for the same shape gives
 * chunks_per_cut and ncuts; saved as in cott_causal_fwd_save, holding sums of k_hat^T v_hat): the backward of the
 * block is then cott_causal_bwd_saved(_bnhd) on q_hat, k_hat, v_hat followed by cott_prep_ex_bwd. */
COTT_API int cott_causal_fwd_prep_save(const void *q, const void *k, const void *v, void *o,
                              void *q_out, void *k_out, void *v_out,
                              const unsigned char *keep, const float *cnt, const float *sig,
                              const float *rot_table, const long long *pos_ids, long long pos0, int rotary_dim,
                              int table_rows, int in_bnhd, int o_bnhd,
                              float *saved, int chunks_per_cut, int ncuts,
                              int B, int H, int N, int Dk, int Dv, int dtype,
                              void *workspace, size_t workspace_bytes, void *stream);

/* ---- per-kernel timing -----------------------------------------------------------------------
 * While enabled, every kernel launch made by the entry points above is bracketed by a pair of HIP
 * events on the launch stream (this is the one place the library creates HIP objects).
 * cott_profile_read() waits for the recorded launches of one kernel family, returns their summed
 * duration and count, and forgets them.  Kernel ids: 0 group_state, 1 state_prefix, 2 causal scan
 * (forward launch), 3 non-causal apply, 4 causal scan (the launch that computes dQ, dK and dV together),
 * 5 generic scan, 6 decode, 7 input preparation, 8 the streaming probe below.  Stands where the reference wraps
 * its kernel call in torch.autograd.profiler (Cuda_Kernel/Custom_Kernel.py:165-179). */
COTT_API int cott_profile_enable(int on);
COTT_API int cott_profile_read(int kernel_id, double *total_ms, long *launches);
COTT_API const char *cott_kernel_name(int kernel_id);

/* ---- launch plans (pure host functions, for tests and tools) -----------------------------------
 * No counterpart in the reference.  The launch plans depend on the device's CU and XCD counts (asked once per process;
 * 256 / 8 when no device answers).  cott_plan_geometry(cus, xcds) replaces them for every later call of this process
 * (0, 0: back to the device's), so that the plans of another part can be examined on any host; cus must be a multiple of xcds.
 * cott_plan_describe: the launches behind `which` = 0 causal forward, 1 causal gradients (with_saved_states: as
 * cott_causal_bwd_saved runs them where cott_causal_saved_plan has a plan), 2 non-causal forward, 3 non-causal
 * gradients, for a shape: *nsets launches (at most 8; 0 when the shape takes the plain-FMA path) and per launch eight
 * ints in sets[8 * s ..]: ops, column halves, sequence groups G, chunks per group, pieces of the group-state pass,
 * whether dK and dV share pair workgroups, whether ops that sum over the past run in complement form, and the
 * workgroups of the scan's grid. */
COTT_API int cott_plan_geometry(int cus, int xcds);
COTT_API int cott_plan_describe(int which, int with_saved_states, int B, int H, int N, int Dk, int Dv, int dtype,
                                int *sets, int *nsets);

/* ---- streaming probe (measurement aid) ---------------------------------------------------------
 * No counterpart in the reference.  Launches a kernel with the launch shape of the scan kernels and none of their
 * arithmetic: `workgroups` workgroups of 256 threads, each walking its own contiguous share of n_read tensors
 * (in + t * tensor_bytes) in blocks of block_bytes (4096, 8192 or 16384) with two blocks of every tensor in flight,
 * and writing its share of n_write tensors (out + t * tensor_bytes).  (n_read, n_write) is (3, 1), a forward pass, or
 * (4, 3), the gradients; tensor_bytes a multiple of workgroups * block_bytes.  The benchmark times it through
 * cott_profile_read beside the kernels to show what the memory system alone needs for a launch of that shape. */
COTT_API int cott_stream_probe(const void *in, void *out, size_t tensor_bytes, int n_read, int n_write, int workgroups,
                               int block_bytes, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* COTTENTION_H */
