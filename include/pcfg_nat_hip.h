/*
 * C-ABI of libpcfg_nat_hip.so: the MI355X (gfx950) implementation of PCFG-NAT's structured-loss hot path.
 *
 * Each entry point replaces one function of the reference's native module
 * (fs_plugins/custom_ops/pcfg_loss.cpp:76-81, declarations :6-18) on raw device pointers: no torch types, no
 * allocation of outputs (the caller owns every buffer), kernels are enqueued on the given HIP stream and the
 * call returns without synchronising unless stated otherwise.
 *
 * Conventions
 *   - `stream` is a hipStream_t passed as void* (NULL = the legacy default stream).
 *   - every function returns PCFGNAT_OK (0) or an error code; pcfgnat_last_error() then holds a message
 *     (thread-local).  Numerical failure (a sentence whose log-likelihood is -inf) is not an error.
 *   - B = batch, L = graph size (decoder positions), T = padded target length, V = vocabulary,
 *     ml = links.size(2) - 1 ("max_left"), Mc = (L-2)/(ml+1)+1 main-chain nodes, Lq = L/4.
 *   - PCFG tables are float32 (the `_f64` entry points take float64 tables, which the reference also dispatches,
 *     pcfg_loss.cu:395), lengths are int64, like every caller in the reference.
 *   - state: the entry points keep nothing between calls except a per-device cache of kernel attributes (and the
 *     process-wide test and tuning settings of pcfg_nat_hip_testing.h, which no call needs).
 */
#ifndef PCFG_NAT_HIP_H
#define PCFG_NAT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PCFGNAT_OK 0
#define PCFGNAT_EINVAL 1       /* argument out of contract */
#define PCFGNAT_EUNSUPPORTED 2 /* valid in the reference but not built here */
#define PCFGNAT_EHIP 3         /* a HIP runtime call failed */

#define PCFGNAT_F16 0
#define PCFGNAT_F32 1
#define PCFGNAT_F64 2

/* ABI version of this header (bumped on incompatible change). */
int pcfgnat_abi_version(void);

/* Message of the last error raised on the calling thread ("" if none). */
const char *pcfgnat_last_error(void);

/*
 * Replaces logsoftmax_gather (logsoftmax_gather.cu:295-359).
 *   word_ins_out [B,L,V] contiguous, dtype PCFGNAT_F16 / F32 / F64.
 *   select_idx   int64, logical shape [B,L,T], element strides (sb, sl, st); the criterion passes a
 *                stride-0 expanded view of the [B,T] targets (nat_pcfg_loss.py:109).
 *   selected     [B,L,T] contiguous, float32 (float64 when dtype is F64):
 *                selected[b,p,s] = word_ins_out[b,p,idx] - max_v - log sum_v exp(. - max_v).
 *   require_grad != 0: word_ins_out is overwritten in place with softmax(word_ins_out) in its own dtype.
 */
int pcfgnat_logsoftmax_gather(void *word_ins_out, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl,
                              int64_t st, void *selected, int require_grad, int64_t B, int64_t L, int64_t V,
                              int64_t T, void *stream);

/*
 * logsoftmax_gather with the criterion's eos mask folded into the gather (nat_pcfg_loss.py:111-115, 201-207):
 * selected[b, p, target_length[b]-1] = -inf for every node p != output_length[b]-1.  Same as calling
 * pcfgnat_logsoftmax_gather and then masked_fill, without the extra passes over [B,L,T].
 */
int pcfgnat_logsoftmax_gather_eos(void *word_ins_out, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl,
                                  int64_t st, void *selected, int require_grad, const int64_t *output_length,
                                  const int64_t *target_length, int64_t B, int64_t L, int64_t V, int64_t T,
                                  void *stream);

/*
 * Replaces the two torch calls of DagLogsoftmaxGatherFunc.backward (pcfg_loss.py:176-177) by one pass:
 *   probs_inout[b,p,v] = probs[b,p,v] * cast(-sum_s g[b,p,s]);  probs_inout[b,p,idx[b,p,s]] += cast(g[b,p,s])
 * with every operation rounded to the buffer's dtype as torch's mul_/scatter_add_ do (duplicates of an index are
 * accumulated in ascending s).  grad_selected is float32 (float64 when dtype is F64), contiguous [B,L,T].
 */
int pcfgnat_logsoftmax_gather_backward(void *probs_inout, int dtype, const int64_t *select_idx, int64_t sb,
                                       int64_t sl, int64_t st, const void *grad_selected, int64_t B, int64_t L,
                                       int64_t V, int64_t T, void *stream);

/*
 * The same pair with the work split differently (no counterpart in the reference, whose forward always overwrites the
 * logits, logsoftmax_gather.cu:238-292): the forward only reads word_ins_out and also returns the log-sum-exp of every
 * row, lse [B,L] (float32; float64 when dtype is F64); the backward turns the untouched logits into the gradient in place,
 *   logits_inout[b,p,v] = -exp(logits[b,p,v] - lse[b,p]) * sum_s g[b,p,s];  logits_inout[b,p,idx[b,p,s]] += g[b,p,s],
 * computed in float32 (float64) and rounded to the buffer's dtype once.  Three passes over the logits per training step
 * instead of four.  output_length/target_length: both NULL, or the lengths for the eos mask of
 * pcfgnat_logsoftmax_gather_eos.
 */
int pcfgnat_logsoftmax_gather_lse(const void *word_ins_out, int dtype, const int64_t *select_idx, int64_t sb, int64_t sl,
                                  int64_t st, void *selected, void *lse, const int64_t *output_length,
                                  const int64_t *target_length, int64_t B, int64_t L, int64_t V, int64_t T, void *stream);
int pcfgnat_logsoftmax_gather_backward_lse(void *logits_inout, int dtype, const int64_t *select_idx, int64_t sb,
                                           int64_t sl, int64_t st, const void *grad_selected, const void *lse, int64_t B,
                                           int64_t L, int64_t V, int64_t T, void *stream);

/*
 * Decode front-end (glat_decomposed_with_link_two_hands_tri_pcfg.py:414-415: log_softmax followed by max over the
 * vocabulary) in one read of the logits: best_lprob[b,p] = max_v logits[b,p,v] - log sum_v exp(logits[b,p,v]) (float32;
 * float64 when dtype is F64), best_idx[b,p] = the first v that attains it (int64).  logits [B,L,V] contiguous.
 */
int pcfgnat_logsoftmax_max(const void *logits, int dtype, void *best_lprob, int64_t *best_idx, int64_t B, int64_t L,
                           int64_t V, void *stream);

/* Number of floats of the auxiliary table the inside kernels exchange (takes the place of the reference's C
 * table, pcfg_loss.cu:394, whose content for ml = 1 is a copy of match_all).  The buffer must be aligned to 16 bytes
 * (the entry points check it where they rely on it). */
size_t pcfgnat_pcfg_aux_floats(int64_t B, int64_t L, int64_t T, int64_t ml);

/*
 * Replaces pcfg_loss (pcfg_loss.cu:379-401): the inside algorithm.
 *   match_all [B,L,T], links [B,L,ml+1,L] contiguous float32 log-probabilities (-inf allowed).
 *   output_length, target_length [B] int64 on the device.
 *   S   [B,Mc,T+2] out: suffix table of main-chain nodes, -inf where undefined; log-likelihood = S[b,0,0].
 *   aux [pcfgnat_pcfg_aux_floats] out: opaque, consumed by the backward and best-tree entry points.
 * Precondition checked on the device per sentence (violations yield S[b,0,0] = NaN, never a fault):
 *   4 <= m <= L, (m-2) % (ml+1) == 0, 2 <= n <= T.
 */
int pcfgnat_pcfg_loss(const float *match_all, const float *links, const int64_t *output_length,
                      const int64_t *target_length, float *S, float *aux, int64_t B, int64_t L, int64_t T,
                      int64_t ml, void *stream);

/*
 * Replaces pcfg_loss_backward (pcfg_loss_backward.cu:654-721): gradients of sum_b grad_output[b] * S[b,0,0].
 *   grad_output [B] float32, or NULL for the criterion's own weights -1/(target_length[b]*B), i.e. the gradient of
 *   loss = -(ll/target_length).mean() (nat_pcfg_loss.py:135); S, aux as produced by pcfgnat_pcfg_loss on the same inputs.
 *   match_all_grad [B,L,T], links_grad [B,L,ml+1,L] out (fully written, zeros outside the support).
 * The result is the exact gradient of the forward recurrences; sentences with a non-finite log-likelihood get
 * all-zero gradients.
 */
int pcfgnat_pcfg_loss_backward(const float *grad_output, const float *S, float *aux, const float *match_all,
                               const float *links, const int64_t *output_length, const int64_t *target_length,
                               float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T,
                               int64_t ml, void *stream);

/*
 * pcfgnat_pcfg_loss followed by pcfgnat_pcfg_loss_backward (same arguments and results: S, match_all_grad, links_grad)
 * in one call.  For max_left = 1 and graphs of up to 128 nodes whose tables fit in LDS (every shipped training shape) the
 * inside and the outside sweep of a sentence run side by side as two workgroups of one launch - the outside recurrence
 * depends on links, emissions and its own earlier columns only, not on the inside table - and a second launch multiplies
 * their tables into the gradients; graphs of 130..1026 nodes are swept by two pipelines of workgroups per sentence,
 * forward and outside, side by side in one launch (see pcfgnat_pipeline_config); otherwise the sweeps follow each other as
 * in the two calls.  aux (pcfgnat_pcfg_aux_floats floats) carries the tables between the launches.
 * For max_left = 3 (--left-tree-layer 2; general loops pcfg_loss.cu:148-214, 262-349) and shapes for which
 * pcfgnat_max_left3_supported answers 1, the sentences whose links hold no rule of a composite local tree - every sentence
 * the model's link scorer can produce: it allows main-chain nodes only as right children
 * (glat_decomposed_with_link_two_hands_tri_pcfg.py:175) - are served by one launch with all tables in LDS; any other
 * sentence of the batch, and every other max_left, by the plain kernels of the two calls.
 */
int pcfgnat_pcfg_loss_forward_backward(const float *grad_output, const float *match_all, const float *links,
                                       const int64_t *output_length, const int64_t *target_length, float *S, float *aux,
                                       float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T, int64_t ml,
                                       void *stream);

/* 1 when pcfgnat_pcfg_loss_forward_backward serves max_left = 3 at this graph size and target length with its one-launch
 * kernel (graphs of up to 254 nodes, targets of up to 64 tokens), 0 when the plain kernels run. */
int pcfgnat_max_left3_supported(int64_t L, int64_t T);

/*
 * No counterpart in the reference: pcfgnat_pcfg_loss_forward_backward for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  Same arguments and results
 * without `aux`: the auxiliary table lives in a device array of PCFGNAT_STATIC_AUX_FLOATS floats (32 MiB) that the library
 * holds on every GPU it is loaded on until the process ends.  The call allocates nothing.  Shapes with
 * pcfgnat_pcfg_aux_floats(B, L, T, ml) > PCFGNAT_STATIC_AUX_FLOATS are rejected with PCFGNAT_EINVAL before anything is
 * enqueued (BASELINE-sized batches fit: 40 sentences of 128 nodes take 2 MiB, 8 of 512 nodes with 140 target tokens
 * 24 MiB).  All calls on one GPU share that GPU's array: calls that overlap there (two streams, two threads) race, and
 * the kernels of one call must have finished before the next call on another stream is enqueued.
 * The first call on a device looks up the array's address and sets kernel attributes (hipGetSymbolAddress,
 * hipFuncSetAttribute), which a stream capture may refuse: make one call per device and shape outside a capture first.
 */
#define PCFGNAT_STATIC_AUX_FLOATS (8u * 1024u * 1024u)
size_t pcfgnat_static_aux_floats(void);
int pcfgnat_pcfg_loss_forward_backward_static(const float *grad_output, const float *match_all, const float *links,
                                              const int64_t *output_length, const int64_t *target_length, float *S,
                                              float *match_all_grad, float *links_grad, int64_t B, int64_t L, int64_t T,
                                              int64_t ml, void *stream);

/*
 * The float64 instantiation the reference also dispatches (AT_DISPATCH_FLOATING_TYPES in pcfg_loss.cu:395,
 * pcfg_loss_backward.cu:693, pcfg_best_tree.cu:349, pcfg_viterbi.cu:291; no shipped script uses it).  Same arguments,
 * layouts and results as the float32 entry points above and below with double tables; every max_left, 1 included,
 * runs the plain one-workgroup-per-sentence kernels, so these are for checking, not for speed.  grad_output is required
 * (no NULL shorthand).  aux holds pcfgnat_pcfg_aux_elems_f64 doubles.
 */
size_t pcfgnat_pcfg_aux_elems_f64(int64_t B, int64_t L, int64_t T, int64_t ml);
int pcfgnat_pcfg_loss_f64(const double *match_all, const double *links, const int64_t *output_length,
                          const int64_t *target_length, double *S, double *aux, int64_t B, int64_t L, int64_t T, int64_t ml,
                          void *stream);
int pcfgnat_pcfg_loss_backward_f64(const double *grad_output, const double *S, double *aux, const double *match_all,
                                   const double *links, const int64_t *output_length, const int64_t *target_length,
                                   double *match_all_grad, double *links_grad, int64_t B, int64_t L, int64_t T, int64_t ml,
                                   void *stream);
int pcfgnat_pcfg_best_tree_f64(const double *S, double *aux, const double *match_all, const double *links,
                               const int64_t *output_length, const int64_t *target_length, int64_t *tree, int64_t B, int64_t L,
                               int64_t T, int64_t ml, void *stream);
int pcfgnat_pcfg_viterbi_f64(const double *ob_lprob, const double *links, const int64_t *output_length, double *S, int64_t *R,
                             int64_t *Lt, int64_t *M, int64_t B, int64_t L, int64_t ml, void *stream);

/*
 * The criterion's reduction (nat_pcfg_loss.py:123-135) on the device: out[0] = -(1/B) sum_b ll_b/target_length[b] over
 * sentences with a finite ll_b = S[b,0,0]; out[1] = number of sentences with a non-finite ll_b.  Deterministic.
 */
int pcfgnat_criterion_loss(const float *S, const int64_t *target_length, float *out, int64_t B, int64_t L, int64_t T,
                           int64_t ml, void *stream);

/*
 * One call for the criterion's whole training pass (nat_pcfg_loss.py:98-145 plus the backward autograd derives from it):
 * logsoftmax_gather with eos mask (log-sum-exp split, see pcfgnat_logsoftmax_gather_lse) -> inside forward -> inside
 * backward with weights -1/(target_length*B) -> logsoftmax_gather backward -> loss.  targets is the contiguous [B,T] int64 target matrix (the gather index of every
 * graph node).  On return (stream order) logits holds d loss / d logits, links_grad d loss / d links, loss_out[0] the
 * loss, loss_out[1] the number of invalid sentences; match_all, S, aux, match_all_grad and row_lse ([B,L] float32) are
 * caller workspaces of the shapes documented at the individual entry points.
 * The rows of the pad nodes at or beyond a sentence's output_length feed nothing in this pass (no sweep reads their
 * gathered values, their gradient is zero): their logits are never read - the gather leaves zeros in match_all and
 * row_lse for them, and the backward writes their gradient rows as zeros - so a step moves the bytes of the live rows
 * three times and those of the pad rows once.
 * matchmask [B,T,L] / keep_word_mask [B,L] (bytes, 0 = false; both NULL = off): the criterion's force-emit masking
 * (nat_pcfg_loss.py:116-121) with the outputs of the glancing step - a graph node whose input was revealed
 * (keep_word_mask) may only emit the target position it is aligned to (matchmask), through a detached value, i.e. the
 * logits row of such a node gets a zero gradient.
 * loss_scale, loss_scale_dev: the factor the caller's loss carries downstream of this criterion (nat_pcfg_loss.py:139-140
 * `loss * factor`, times the fp16 loss scale of every shipped training script): a host value times an optional float32
 * scalar in device memory (NULL = 1).  Both gradients come out multiplied by it; it enters the weights -1/(target_length*B)
 * in float32, i.e. ahead of the single rounding of d loss / d logits to the logits' dtype, as in pcfg_loss.py:77-83, 176-177.
 * loss_out[0] stays the unscaled loss.
 * events: NULL, or six hipEvent_t (entries may be NULL) recorded before/after the gather forward, the inside
 * forward+backward and the gather backward (for timing).
 */
int pcfgnat_criterion_step(void *logits, int dtype, const int64_t *targets, const float *links,
                           const int64_t *output_length, const int64_t *target_length, const unsigned char *matchmask,
                           const unsigned char *keep_word_mask, float *match_all, float *S,
                           float *aux, float *match_all_grad, float *links_grad, float *row_lse, float *loss_out, int64_t B,
                           int64_t L, int64_t V, int64_t T, int64_t ml, float loss_scale,
                           const float *loss_scale_dev, void *stream, void *const *events);

/*
 * The same pass cut where autograd cuts it (no counterpart in the reference, which leaves the cut to torch:
 * pcfg_loss.py:67-83 saves the inside gradients in the forward and scales them by grad_output in the backward,
 * :176-177 scale the probabilities by the upstream gradient before they are cast to the logits' dtype).
 *   forward:  gather with eos mask (read only) -> inside forward + backward with weights -1/(target_length*B) -> loss.
 *             Leaves match_all_grad, links_grad (both at an upstream gradient of 1), row_lse, loss_out[0..1] and, where ll_out
 *             is not null, ll_out [B] = the log-likelihoods with those of invalid sentences zeroed (nat_pcfg_loss.py:123-133);
 *             the logits are untouched except that the rows of pad nodes may already be zeroed (*pad_rows_zeroed tells, pass
 *             it on).
 *   backward: logits_inout becomes upstream * d loss / d logits in one read + write pass, links_grad_inout is multiplied by
 *             upstream by the threads of the same launch.  upstream_dev: one float32 in device memory (the gradient flowing into the loss, e.g. the fp16 loss
 *             scale times the criterion's factor; NULL = 1).  It multiplies the emission posteriors in float32 ahead of the
 *             single rounding to the logits' dtype, so gradients below the fp16 range at scale 1 survive, and no value ever
 *             passes through the host.
 */
int pcfgnat_criterion_forward(void *logits, int dtype, const int64_t *targets, const float *links, const int64_t *output_length,
                              const int64_t *target_length, const unsigned char *matchmask, const unsigned char *keep_word_mask,
                              float *match_all, float *S, float *aux, float *match_all_grad, float *links_grad, float *row_lse,
                              float *loss_out, float *ll_out, int *pad_rows_zeroed, int64_t B, int64_t L, int64_t V, int64_t T,
                              int64_t ml, void *stream);
int pcfgnat_criterion_backward(void *logits_inout, int dtype, const int64_t *targets, const float *match_all_grad,
                               const float *row_lse, const unsigned char *keep_word_mask, const int64_t *output_length,
                               int pad_rows_zeroed, const float *upstream_dev, float *links_grad_inout, int64_t B, int64_t L,
                               int64_t V, int64_t T, int64_t ml, void *stream);

/*
 * The link scorer of the model (glat_decomposed_with_link_two_hands_tri_pcfg.py:140-201, `extract_links`) after its four
 * projections, for max_left = 1:
 *   links[b,a,k,c] = logsumexp_h( log_softmax_h(gate_logits[b,a,:])[h] + log_softmax_{(k,c)}( z[b,a,:,:,h] )[k,c] ),
 *   z[b,a,k,c,h] = ( q[b,a,h].kl[b,left(a,k),h] + kl[b,src(a,k),h].kr[b,c,h] + q[b,a,h].kr[b,c,h] ) / sqrt(F),
 * left(a,0) = src(a,0) = 0, left(a,1) = max(a-1,0), src(a,1) = a-1 cyclically; masked entries (:171-184) and rows
 * without an allowed left option or right child (:176-181, 199) are -inf.  The batched products go through the
 * caller's GEMM library; the five calls are, in order:
 *   pack:     query/left-key/right-key chunks [B,L,H,F] (F16/F32/F64) -> A [B,H,2L,F] (query rows, then left-key rows) and
 *             Kr [B,H,L,F], float32.                      Caller: Z = A . Kr^T  [B,H,2L,L].
 *   forward:  Z, A, gate_logits [B,L,H] float32, prev_output_tokens [B,L] int64, left_tree_mask / right_tree_mask [L,L]
 *             and main_chain [L] (one byte per flag; masks: non-zero = forbidden) -> links [B,L,2,L], head_lse [B,L,H].
 *   backward: grad_links, links, head_lse, Z, A, ... -> dZ [B,H,2L,L] (gradient of Z, complete), dZ0 [B,H,L,L] (scratch),
 *             dsab [B,H,L,2] (gradient of the two q.kl dot products of every parent), dgate [B,L,H] (gradient of the
 *             gate logits).                               Caller: dA = dZ . Kr, dKr = dZ^T . A.
 *   unpack:   dA, dKr, dsab, A -> gradients of the three chunk tensors [B,L,H,F] in `dtype`.
 * Nothing of size [B,L,2L,H] is materialised in either direction.
 */
int pcfgnat_extract_links_pack(const void *query_chunks, const void *key_chunks_left, const void *key_chunks_right, int dtype,
                               float *A, float *Kr, int64_t B, int64_t L, int64_t H, int64_t F, void *stream);
int pcfgnat_extract_links_forward(const float *Z, const float *A, const float *gate_logits, const int64_t *prev_output_tokens,
                                  int64_t pad_index, const unsigned char *left_tree_mask, const unsigned char *right_tree_mask,
                                  const unsigned char *main_chain, float *links, float *head_lse, int64_t B, int64_t L,
                                  int64_t H, int64_t F, void *stream);
int pcfgnat_extract_links_backward(const float *grad_links, const float *links, const float *head_lse, const float *Z,
                                   const float *A, const float *gate_logits, const int64_t *prev_output_tokens,
                                   int64_t pad_index, const unsigned char *left_tree_mask,
                                   const unsigned char *right_tree_mask, const unsigned char *main_chain, float *dZ, float *dZ0,
                                   float *dsab, float *dgate, int64_t B, int64_t L, int64_t H, int64_t F, void *stream);
int pcfgnat_extract_links_unpack(const float *dA, const float *dKr, const float *dsab, const float *A, int dtype, void *dq,
                                 void *dkl, void *dkr, int64_t B, int64_t L, int64_t H, int64_t F, void *stream);

/*
 * The same scorer (same reference lines) with the three products inside the kernels, on the matrix cores: one call
 * forward, nothing for the caller to multiply.  Built for float16 chunks with F a multiple of 16 up to 128 and float32
 * chunks with F a multiple of 8 up to 64, as long as the rows of a 32-parent tile fit the local memory
 * (pcfgnat_extract_links_fused_supported returns 1; otherwise the calls return PCFGNAT_EUNSUPPORTED and the five-call
 * form above applies).  Chunks [B,L,H,F] contiguous and 16-byte aligned, the other arguments as above.
 *   fused_forward:  -> links [B,L,2,L], head_lse [B,L,H] and, where tile_masks is not null, tile_masks [B,L,1+ceil(L/32)]
 *                   (per parent a word of flags and its allowed right children as bits; what the backward reads).
 *   fused_backward: grad_links, links, head_lse, tile_masks as the forward left them, and the chunks and gate logits
 *                   of the forward -> gradients of the three chunk tensors [B,L,H,F] in `dtype` and of the gate logits
 *                   [B,L,H] float32, in three launches; built for head dimensions up to 64 (fused_backward_supported
 *                   returns 1).  workspace: device memory of fused_backward_workspace_bytes(B, L, H, F) bytes, 16-byte
 *                   aligned, contents irrelevant on entry.
 */
int pcfgnat_extract_links_fused_supported(int dtype, int64_t L, int64_t H, int64_t F);
int pcfgnat_extract_links_fused_forward(const void *query_chunks, const void *key_chunks_left, const void *key_chunks_right, int dtype,
                                        const float *gate_logits, const int64_t *prev_output_tokens, int64_t pad_index,
                                        const unsigned char *left_tree_mask, const unsigned char *right_tree_mask,
                                        const unsigned char *main_chain, float *links, float *head_lse, unsigned *tile_masks,
                                        int64_t B, int64_t L, int64_t H, int64_t F, void *stream);
int pcfgnat_extract_links_fused_backward_supported(int dtype, int64_t L, int64_t H, int64_t F);
size_t pcfgnat_extract_links_fused_backward_workspace_bytes(int64_t B, int64_t L, int64_t H, int64_t F);
int pcfgnat_extract_links_fused_backward(const float *grad_links, const float *links, const float *head_lse,
                                         const unsigned *tile_masks, const void *query_chunks, const void *key_chunks_left,
                                         const void *key_chunks_right, int dtype, const float *gate_logits, void *dq, void *dkl,
                                         void *dkr, float *dgate, float *workspace, int64_t B, int64_t L, int64_t H, int64_t F,
                                         void *stream);

/*
 * GLAT glancing (nat_pcfg_loss.py:193-269) in one call: lengths from the pad counts
 * (:195-196), arg max of the logits (:199), logsoftmax_gather without gradient + eos mask (:200-207), best-tree alignment
 * (:210), and everything the criterion derives from the alignment (:212-255), for each of its glance strategies:
 * PCFGNAT_GLANCE_NUMBER_RANDOM (`number-random`, :235-242, every shipped script), PCFGNAT_GLANCE_CMLM (`cmlm`, :244-251),
 * PCFGNAT_GLANCE_DEFAULT (no strategy named, :231-233).
 *   logits [B,L,V] (F16/F32/F64, read only); targets [B,T], prev_output_tokens [B,L] int64; links [B,L,ml+1,L] float32;
 *   the caller's random draws, float32, made in the reference's order: noise [B,L] = randn (:235 / :245; number-random and
 *   cmlm, else may be null), length_rand [B] = rand (:247; cmlm only, else may be null), keep_rand [B,L] = rand (:253; read
 *   by the default strategy only - with the other two keep_prob is 0 or 1 and the draw cannot change the result, the
 *   caller still makes it to keep its random stream in step - may be null for them); context_p: glancing ratio.
 * Workspaces: match_all [B,L,T], S [B,Mc,T+2], aux [pcfgnat_pcfg_aux_floats] float32; pred_tokens [B,L], lengths [2,B] int64
 * (the logits of pad nodes at or beyond a sentence's output length are not read: zeros in match_all and pred_tokens).
 * Outputs: path [B,L] int64 (target position of every node, -1 off the tree); matchmask [B,T,L], keep_word_mask [B,L]
 * (one byte per flag, 0/1); glat_prev_output_tokens [B,L], same_num [B], glance_nums [B] int64 (zeros for the default
 * strategy, which has none); loss_out[0] =
 * -(ll/target_length).mean() over sentences with a finite best-tree likelihood ll = S[b,0,0], loss_out[1] = number of
 * the others.  On return lengths[0,:] = output_length and lengths[1,:] = target_length.
 */
#define PCFGNAT_GLANCE_NUMBER_RANDOM 0
#define PCFGNAT_GLANCE_CMLM 1
#define PCFGNAT_GLANCE_DEFAULT 2
int pcfgnat_glat_step(const void *logits, int dtype, const int64_t *targets, const int64_t *prev_output_tokens,
                      const float *links, int glance_strategy, const float *noise, const float *length_rand,
                      const float *keep_rand, float context_p, int64_t pad_index, float *match_all, float *S,
                      float *aux, int64_t *pred_tokens, int64_t *lengths, int64_t *path, unsigned char *matchmask,
                      unsigned char *keep_word_mask, int64_t *glat_prev_output_tokens, int64_t *same_num,
                      int64_t *glance_nums, float *loss_out, int64_t B, int64_t L, int64_t V, int64_t T, int64_t ml,
                      void *stream);

/*
 * Replaces pcfg_best_tree (pcfg_best_tree.cu:333-360): greedy top-down trace over the inside tables.
 *   tree [B,L] int64 out: target position aligned to each node, -1 for nodes off the tree.
 * Exact ties are resolved in the reference's scan order (lanes 0 > 2 > 1 > 3 of a 4-wide strided scan).
 * aux: the table left by pcfgnat_pcfg_loss on the same inputs (read, and for max_left != 1 partly reused as mark space).
 */
int pcfgnat_pcfg_best_tree(const float *S, float *aux, const float *match_all, const float *links,
                           const int64_t *output_length, const int64_t *target_length, int64_t *tree, int64_t B,
                           int64_t L, int64_t T, int64_t ml, void *stream);

/*
 * Replaces pcfg_viterbi (pcfg_viterbi.cu:272-301): max-product tables per output length.
 *   ob_lprob [B,L] float32, links [B,L,ml+1,L] float32, output_length [B] int64.
 *   S [B,L,Lq] float32 out (-inf where undefined; the Python wrapper returns row 1),
 *   R, Lt, M [B,L,Lq] int64 out (right child, left child, left span; 0 where undefined).
 * Values and arg-max decisions are bit-identical to a sequential fp32 evaluation in the reference's order.
 */
int pcfgnat_pcfg_viterbi(const float *ob_lprob, const float *links, const int64_t *output_length, float *S,
                         int64_t *R, int64_t *Lt, int64_t *M, int64_t B, int64_t L, int64_t ml, void *stream);

/*
 * Replaces viterbi_decoding (pcfg_loss.cpp:12-73) for traces that live on the device: one walk per sentence.
 *   pred_length, output_length [B] int64; Lt, R, M [B,L,Lq] int64; tokens [B,L] int64;
 *   left_tree_mask [mask_dim,mask_dim] int64 (non-zero = forbidden).
 *   out_tokens [B,L] int64 out: emitted tokens, right-padded with pad_index; out_count [B] int64 out: how many
 *   (-1 for malformed traces); scratch [B,2L] int64: the explicit stacks of the walks.
 */
int pcfgnat_viterbi_decoding(const int64_t *pred_length, const int64_t *output_length, const int64_t *Lt,
                             const int64_t *R, const int64_t *M, const int64_t *tokens,
                             const int64_t *left_tree_mask, int64_t mask_dim, int64_t pad_index,
                             int64_t *out_tokens, int64_t *out_count, int64_t *scratch, int64_t B, int64_t L,
                             int64_t Lq, void *stream);

/*
 * The whole Viterbi decode of glat_decomposed_with_link_two_hands_tri_pcfg.py:483-502 in one call: tables
 * (pcfg_viterbi.cu:272-301), length selection pred_length = 1 + argmax_{len >= 1} S[b,1,len] / length_penalty[len] with NaN
 * read as -inf and the first maximum winning (:489-497), and the walk (pcfg_loss.cpp:12-73).  length_penalty [L/4] float32
 * is the caller's arange(L/4) ** decode_viterbibeta.  For max_left = 1 and graphs of up to 514 nodes the traces are one
 * int32 per cell in `workspace` and the call is a single launch, or - from about 200 nodes on, see pcfgnat_pipeline_config -
 * a sweep by a pipeline of workgroups per sentence followed by the selection and the walk; otherwise the three steps run
 * back to back on full tables in `workspace`.  workspace: pcfgnat_viterbi_decode_workspace_bytes(B, L, max_left) bytes,
 * 8-byte aligned.
 *   out_tokens [B,L] int64, out_count [B] int64 (as pcfgnat_viterbi_decoding), pred_length [B] int64.
 *   out_tokens_f32 [B,L] float32 or NULL: the same rows once more as float32, the type the model hands on (:501 ends in
 *   `.float()`), written by the kernel that walks the tree so that the caller launches no conversion of its own.  A
 *   sentence's out_count is the last thing stored for it.
 */
size_t pcfgnat_viterbi_decode_workspace_bytes(int64_t B, int64_t L, int64_t ml);
int pcfgnat_viterbi_decode(const float *ob_lprob, const float *links, const int64_t *output_length, const int64_t *tokens,
                           const int64_t *left_tree_mask, int64_t mask_dim, int64_t pad_index, const float *length_penalty,
                           void *workspace, int64_t *out_tokens, float *out_tokens_f32, int64_t *out_count,
                           int64_t *pred_length, int64_t B, int64_t L, int64_t ml, void *stream);

/*
 * The decode as the model runs it (glat_decomposed_with_link_two_hands_tri_pcfg.py:414-416 followed by :483-502) enqueued
 * by one call: pcfgnat_logsoftmax_max over logits [B,L,V] (float16 or float32) into best_lprob [B,L] float32 and best_idx
 * [B,L] int64 (both out: the node scores and node tokens of the decode), then pcfgnat_viterbi_decode on them.  The other
 * arguments and the results are those of pcfgnat_viterbi_decode.
 */
int pcfgnat_viterbi_decode_logits(const void *logits, int dtype, int64_t V, float *best_lprob, int64_t *best_idx,
                                  const float *links, const int64_t *output_length, const int64_t *left_tree_mask,
                                  int64_t mask_dim, int64_t pad_index, const float *length_penalty, void *workspace,
                                  int64_t *out_tokens, float *out_tokens_f32, int64_t *out_count, int64_t *pred_length,
                                  int64_t B, int64_t L, int64_t ml, void *stream);

/*
 * The `lookahead` and `greedy` decode strategies of glat_decomposed_with_link_two_hands_tri_pcfg.py:419-481 in one launch:
 * per node the first arg max over (k, c) of (links[b,a,k,c] + ob[b,c]*beta) + ob[b,left(a,k)]*beta (lookahead; ob_lprob
 * NULL selects greedy: links alone), then the in-order walk from node 1 over these pointers.  The reference builds the
 * left term from sentence 0's logits for every sentence of a batch (:424, a batch-1 routine); the per-sentence term is
 * used here.  Tokens are not de-duplicated (unlike pcfgnat_viterbi_decoding).
 *   links_idx [B,L] int64 out (may be NULL): k*L + c per node; out_tokens [B,L] int64, right-padded with pad_index;
 *   out_count [B] int64 (-1 if a walk does not terminate).
 */
int pcfgnat_lookahead_decode(const float *links, const float *ob_lprob, float beta, const int64_t *output_length,
                             const int64_t *tokens, const int64_t *left_tree_mask, int64_t mask_dim, int64_t pad_index,
                             int64_t *links_idx, int64_t *out_tokens, int64_t *out_count, int64_t B, int64_t L, int64_t ml,
                             void *stream);

/* The same walk on host memory (the reference's own call site hands over CPU tensors,
 * glat_decomposed_with_link_two_hands_tri_pcfg.py:500-502).  Synchronous, touches no GPU. */
int pcfgnat_viterbi_decoding_host(const int64_t *pred_length, const int64_t *output_length, const int64_t *Lt,
                                  const int64_t *R, const int64_t *M, const int64_t *tokens,
                                  const int64_t *left_tree_mask, int64_t mask_dim, int64_t pad_index,
                                  int64_t *out_tokens, int64_t *out_count, int64_t B, int64_t L, int64_t Lq);

#ifdef __cplusplus
}
#endif
#endif /* PCFG_NAT_HIP_H */
