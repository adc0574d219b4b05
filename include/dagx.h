/*
 * dagx -- C ABI of the MI355X (gfx950) DAG training operators.
 *
 * This is the boundary a DA-Transformer checkout binds instead of its pybind module
 * `dag_loss_fn` (fs_plugins/custom_ops/dag_loss.cpp:19-28).  Plain pointers and sizes only:
 * no torch types, no allocation, no synchronisation.  Every pointer is a device pointer
 * unless stated otherwise; every kernel is enqueued on `stream` (a hipStream_t passed as
 * void*) and the call returns immediately.
 *
 * Return value: DAGX_OK (0) or an error code; dagx_last_error() gives the message of the last
 * failing call made by the calling thread.  Nothing here aborts the process or the GPU context;
 * samples whose lengths admit no path yield loss = -inf, zero gradients and an all -1 path.
 *
 * Layouts (B samples, T = max target length, L = max graph size, V vocabulary,
 * S gathered ids per row, translen = max transition distance):
 *   match      [B,T,L]        any element strides, dtype f32/f16/bf16   log P(target t | node j)
 *   links      [B,L,translen] contiguous ("shifted": entry [i,d] = log P(i -> i+d+1); -inf = no edge)
 *   out_len, tgt_len  [B] int64 (L_b, T_b)
 */
#ifndef DAGX_H_
#define DAGX_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { DAGX_F32 = 0, DAGX_F16 = 1, DAGX_BF16 = 2 };

enum {
    DAGX_OK = 0,
    DAGX_ERR_ARGUMENT = 1,     /* null pointer, negative size, bad dtype ... */
    DAGX_ERR_UNSUPPORTED = 2,  /* a size beyond what the kernels are built for */
    DAGX_ERR_WORKSPACE = 3,    /* workspace missing or too small */
    DAGX_ERR_LAUNCH = 4        /* HIP reported an error at launch */
};

/* Which operator dagx_workspace_bytes() is asked about. */
enum { DAGX_OP_LOSS_FWD = 0, DAGX_OP_LOSS_BWD = 1, DAGX_OP_BEST_ALIGNMENT = 2, DAGX_OP_VITERBI_DECODE = 3,
       DAGX_OP_BEST_ALIGNMENT_F64 = 4 };

/* Library version string, e.g. "dagx 0.3 (gfx950)".  No reference counterpart. */
const char *dagx_version(void);

/* Message of the last error on this host thread ("" if none).  Replaces the TORCH_CHECK
 * exceptions of fs_plugins/custom_ops/dag_loss.cu:317-332 and logsoftmax_gather.cu:315-327. */
const char *dagx_last_error(void);

/* Process-wide switch: 1 makes dagx_loss_fwd / dagx_loss_bwd / dagx_best_alignment use only
 * their log-domain (one workgroup per sample) kernels, zero (default, or DAGX_EXACT_SWEEP unset)
 * lets them use the tile-resident kernels.  2 is for tests: as zero, but dagx_best_alignment then
 * treats every sample as one that its tile pipeline gave up on, and does it again the way it does
 * those.  Returns the previous setting.  No reference counterpart
 * (the reference's DagLossFunc.config* launch-shape selectors are the closest thing,
 * fs_plugins/custom_ops/dag_loss.py:66-68). */
int dagx_force_log_domain(int on);

/* Process-wide switch for dagx_loss_fwd / dagx_loss_fwd_noalloc: non-zero makes them start with the float64 tile
 * sweeps for every sample instead of trying the float32 ones first (zero: default, or DAGX_FLOAT64_FIRST unset).
 * For callers who know their inputs for long and sharply peaked (a trained model's graphs of a thousand nodes):
 * there the float32 sweeps rarely stand and their pass is lost time; the float64 sweeps cost 1.6 times as much
 * per sample and hold 1300 nats under every scale.  Results keep the same guarantee either way.  Returns the
 * previous setting.  No reference counterpart (the reference's kernels have one speed). */
int dagx_loss_float64_first(int on);

/* Scratch bytes the caller must provide to the given operator (may be 0).  The reference
 * allocates its scratch itself (fs_plugins/custom_ops/dag_loss.cu:154, dag_best_alignment.cu:244-246). */
size_t dagx_workspace_bytes(int op, int B, int T, int L, int translen);

/*
 * Fused log-softmax + gather, forward.  Replaces `logsoftmax_gather`
 * (fs_plugins/custom_ops/dag_loss.cpp:22, bound at :28; logsoftmax_gather.cu:313-377) as called from
 * DagLogsoftmaxGatherFunc.forward (fs_plugins/custom_ops/dag_loss.py:205-214).
 *   logits [B,L,V] contiguous, read only;  idx [B,L,S] int64 with element strides idx_strides[3]
 *   (stride 0 allowed);  sel: float32, element strides sel_strides[3] for the logical [B,L,S]
 *   index (so the caller may ask for a [B,S,L] memory order);  lse: [B*L] float32 or NULL --
 *   log-sum-exp of every row, which is all the backward needs (the logits are NOT overwritten
 *   with probabilities).  Ids outside [0,V) give NaN instead of a fault.
 */
int dagx_lsg_fwd(const void *logits, int dtype, int B, int L, int64_t V, int S,
                 const int64_t *idx, const int64_t idx_strides[3],
                 float *sel, const int64_t sel_strides[3],
                 float *lse, void *stream);

/*
 * Fused log-softmax + gather, backward, in place: logits[b,l,v] <- -softmax(logits[b,l,:])[v] *
 * sum_s g[b,l,s] + sum_{s: idx[b,l,s]=v} g[b,l,s], rounded once to the logits' dtype.  Replaces
 * the mul_/scatter_add_ pair of DagLogsoftmaxGatherFunc.backward
 * (fs_plugins/custom_ops/dag_loss.py:227-231).  grad_sel is float32 with element strides
 * gsel_strides[3] for the logical [B,L,S] index; lse is what dagx_lsg_fwd wrote.
 */
int dagx_lsg_bwd(void *logits_inout, int dtype, int B, int L, int64_t V, int S,
                 const int64_t *idx, const int64_t idx_strides[3],
                 const float *grad_sel, const int64_t gsel_strides[3],
                 const float *lse, void *stream);

/*
 * Transition log-probabilities from per-head scores, forward: the tail of the link predictor,
 * fs_plugins/models/glat_decomposed_with_link.py:380-404 with extract_valid_links (:319-335) --
 * mask, gather into the shifted layout, log_softmax over the transitions, add the gate
 * log-probabilities, logsumexp over the heads -- in one pass (it has no counterpart among the
 * reference's native operators; the reference runs it as a chain of PyTorch calls).
 *   content   [B,L,L,H] contiguous, the dtype given; content[b,i,j,c] = score of i -> j for head c
 *   log_gates [B,L,H] float32;  valid_end [B,L] int64: transitions i -> j are allowed for
 *   i < j < valid_end[b,i] (the number of non-pad nodes, or bound_end + 1)
 *   links     [B,L,translen], same dtype: links[b,i,d] = log P(i -> i+d+1), -inf where not allowed
 *   lse       [B,L,H] float32 or NULL: per-head log normalisers, all the backward needs
 * H is 4, 8 or 16; L <= 1024.
 */
int dagx_links_fwd(const void *content, int dtype, const float *log_gates, const int64_t *valid_end,
                   int B, int L, int H, int translen, void *links, float *lse, void *stream);

/*
 * Backward of dagx_links_fwd, in place: content <- d loss / d content (0 wherever a transition is
 * not allowed), grad_gates [B,L,H] float32 <- d loss / d log_gates.  lse is what the forward wrote,
 * grad_links [B,L,translen] has the dtype of content.  links is not read and may be NULL: the weights of the
 * heads are formed again from the scores in float32 (a link value rounded to bfloat16 would put them 3 % off).
 */
int dagx_links_bwd(void *content_inout, int dtype, const float *log_gates, const int64_t *valid_end,
                   int B, int L, int H, int translen, const void *links, const float *lse,
                   const void *grad_links, float *grad_gates, void *stream);

/*
 * Storage of the sweep results.  Positions are p = node for alpha and p = L_b-1-node for beta, in
 * blocks of 64.  Every (t, block) has a float64 offset and every cell a float32 residual <= 0:
 *     alpha[b][t][node] = alpha_off[b][t][p/64] + alpha_hat[b][t][node]      (same for beta)
 * alpha_hat/beta_hat are [B,T,L] float32, alpha_off/beta_off are [B,T,ceil(L/64)] float64, logz is
 * [2,B] float64 (log-likelihood read from the alpha sweep, then from the beta sweep) and loss [B]
 * is the one the caller gets, in float32: the beta read-out when require_gradient is non-zero (the
 * partition function the backward divides by), the alpha read-out otherwise -- the choice of
 * DagLossFunc.forward (fs_plugins/custom_ops/dag_loss.py:106-109).  Only cells with t < T_b and node < L_b are defined.  sample_flags [B] int32
 * records which kernel's result stands for each sample: 0 the float32 tile sweeps', 2 the float64 ("wide") tile
 * sweeps', 1 the log-domain kernel's (a diagnostic; the tables have one format and the backward does not look).
 *
 * DAG loss forward.
 * workspace: dagx_workspace_bytes(DAGX_OP_LOSS_FWD, ...) bytes, 8-byte aligned.  It MUST BE ZERO-FILLED when it
 * is first handed to this function (dagx_loss_fwd_init_workspace does that; with garbage in it the result is
 * undefined and nothing detects it); every call leaves it zero-filled again (its kernels clear the words they
 * used), so one buffer, cleared once, serves any number of consecutive calls of any shape.  Calls that overlap
 * in time need separate workspaces.
 * With require_gradient non-zero the alpha and the beta sweep run (loss = the beta read-out); otherwise the alpha
 * sweep runs twice and loss is its read-out (beta_hat, beta_off and the second row of logz are then scratch, and
 * dagx_loss_bwd must not be called on the result).  Either way the two sweeps of a sample bracket log Z: the
 * tile kernels work in a scaled linear domain that cannot hold numbers more than 126 nats under their scale; one
 * sweep lets such numbers become 0 (its read-out never exceeds log Z), the other puts the smallest number it
 * holds in their place (its read-out never falls short of it).  A sample whose two read-outs agree stands;
 * any other is swept again with float64 linear-domain numbers (1300 nats of room, two instructions per
 * pair-update instead of one) under the same test, and what that leaves is computed by the log-domain kernel,
 * which has no such limit (and no such speed).
 * Replaces `dag_loss` (fs_plugins/custom_ops/dag_loss.cpp:19, bound at :25;
 * dag_loss.cu:313-375) as called from DagLossFunc.forward (fs_plugins/custom_ops/dag_loss.py:101-111).
 * Setting the environment variable DAGX_EXACT_SWEEP=1 forces the log-domain kernel for every sample.
 */
int dagx_loss_fwd(const void *match, int match_dtype, const int64_t match_strides[3],
                  const void *links, int links_dtype,
                  const int64_t *out_len, const int64_t *tgt_len,
                  int B, int T, int L, int translen,
                  float *alpha_hat, float *beta_hat, double *alpha_off, double *beta_off,
                  double *logz, float *loss, int *sample_flags, int require_gradient,
                  void *workspace, size_t workspace_bytes, void *stream);

/* Zero-fill of a workspace for dagx_loss_fwd: one kernel launch on `stream`, needed once per buffer.  No reference
 * counterpart (the reference allocates zeroed scratch inside every call, dag_loss.cu:339-340). */
int dagx_loss_fwd_init_workspace(void *workspace, size_t workspace_bytes, void *stream);

/* What dagx_loss_fwd and dagx_loss_fwd_noalloc otherwise do on their first call on a device, for the current
 * device: the LDS limit of the tile kernels (hipFuncSetAttribute) and the address of the built-in scratch array
 * (hipGetSymbolAddress).  Neither may be part of a stream capture: a caller that captures these entry points into a
 * HIP graph calls this once per device beforehand (or makes one ordinary call first).  No reference counterpart. */
int dagx_prepare_device(void);

/*
 * dagx_loss_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and
 * results as dagx_loss_fwd but for the workspace: the pipeline words live in a device array of
 * dagx_loss_fwd_noalloc_max_bytes() = 128 KiB that the library owns (one copy per GPU, held until the process
 * ends), so the call allocates nothing, frees nothing and calls no allocating routine.  Shapes whose
 * dagx_workspace_bytes(DAGX_OP_LOSS_FWD, ...) exceed that size are refused with DAGX_ERR_UNSUPPORTED (with
 * B <= 64 every graph size fits; L <= 512 fits up to B = 1024).  All calls on one GPU share the array: calls
 * that overlap in time on one GPU (different streams, or different host threads) race and must be
 * serialised by the caller; consecutive calls on one stream are fine (the kernels leave the array zero, which
 * is the state they need on entry).  Under stream capture: call dagx_prepare_device() once on the device before
 * capturing (the first call on a device otherwise looks up the array's address and raises a kernel's LDS limit,
 * which a capture cannot hold), and keep L <= 3072 (beyond it the log-domain kernel's LDS limit is raised per call).
 */
size_t dagx_loss_fwd_noalloc_max_bytes(void);
int dagx_loss_fwd_noalloc(const void *match, int match_dtype, const int64_t match_strides[3],
                          const void *links, int links_dtype,
                          const int64_t *out_len, const int64_t *tgt_len,
                          int B, int T, int L, int translen,
                          float *alpha_hat, float *beta_hat, double *alpha_off, double *beta_off,
                          double *logz, float *loss, int *sample_flags, int require_gradient,
                          void *stream);

/*
 * DAG loss backward.  Replaces `dag_loss_backward` (fs_plugins/custom_ops/dag_loss.cpp:20, bound at :26;
 * dag_loss.cu:518-571) as called from DagLossFunc.backward (fs_plugins/custom_ops/dag_loss.py:113-120).
 *   grad_out [B] float32 (element stride grad_out_stride);  grad_match [B,T,L] contiguous in
 *   match_dtype;  grad_links [B,L,translen] contiguous in links_dtype.  Either output may be NULL.
 *   The seven pointers after grad_out_stride are what dagx_loss_fwd wrote.
 *   workspace: unused (dagx_workspace_bytes(DAGX_OP_LOSS_BWD, ...) is 0); NULL is fine.
 */
int dagx_loss_bwd(const float *grad_out, int64_t grad_out_stride,
                  const float *alpha_hat, const float *beta_hat,
                  const double *alpha_off, const double *beta_off, const double *logz,
                  const int *sample_flags,
                  const void *match, int match_dtype, const int64_t match_strides[3],
                  const void *links, int links_dtype,
                  const int64_t *out_len, const int64_t *tgt_len,
                  int B, int T, int L, int translen,
                  void *grad_match, void *grad_links,
                  void *workspace, size_t workspace_bytes, void *stream);

/*
 * Viterbi alignment with on-GPU backtrack.  Replaces `dag_best_alignment`
 * (fs_plugins/custom_ops/dag_loss.cpp:21, bound at :27; dag_best_alignment.cu:219-263) as called from
 * DagBestAlignmentFunc.forward (fs_plugins/custom_ops/dag_loss.py:159-164).
 *   path [B,L] int64: target position emitted by node j on the best path, else -1.  Scores are
 *   float32 with two roundings per cell (add, max, add); among equal predecessors the lowest
 *   index wins (the torch-native rule, fs_plugins/custom_ops/dag_loss.py:253-257, 350).
 */
int dagx_best_alignment(const void *match, int match_dtype, const int64_t match_strides[3],
                        const void *links, int links_dtype,
                        const int64_t *out_len, const int64_t *tgt_len,
                        int B, int T, int L, int translen,
                        int64_t *path,
                        void *workspace, size_t workspace_bytes, void *stream);

/*
 * Pinning nodes to targets by rewriting `match`.  Replaces NATDAGLoss._force_aligment
 * (fs_plugins/criterions/nat_dag_loss.py:111-120), a chain of tensor operations over
 * [B,T+1,L] masks, by one launch.
 *   match      [B,T,L] in match_dtype, element strides strides[3]
 *   force_emit [B,L] int64 contiguous: t in [0,T) pins node j to target t, -1 does not
 *   out        [B,T,L] contiguous, same dtype
 * gradient == 0: a target row named by any node becomes 0 at the naming nodes and -inf elsewhere;
 * other rows pass through.  gradient != 0: `match` is the gradient with respect to the rewritten
 * tensor and out the gradient with respect to the original one (named rows 0, others unchanged).
 */
int dagx_force_emit(const void *match, int match_dtype, const int64_t strides[3], const int64_t *force_emit,
                    int B, int T, int L, int gradient, void *out, void *stream);

/*
 * Glancing after the best alignment.  Replaces the tensor operations of glat_function
 * (fs_plugins/criterions/nat_dag_loss.py:273-278 and :307-311) by one launch.  All tensors are
 * contiguous; tokens, path and counts are int64, masks are bytes (0/1).
 *   stages & 1 (oracle): oracle[B,L] = tgt_tokens[b, max(path, 0)];  same_num[B] = assigned, not
 *       pinned nodes whose pred_tokens equal the oracle token (prev_mask [B,L] marks pinned nodes,
 *       NULL = none)
 *   stages & 2 (mix): keep_mask = rand < keep_prob or pinned;  glat_tokens = keep ? oracle :
 *       prev_output_tokens;  next_force_emit = keep ? path : -1.  With keep_prob_in == NULL (needs
 *       stages == 3) the keep probability is that of glance_strategy None,
 *       ((T_b - pinned - same_num) / T_b * context_p) on assigned nodes and 0 elsewhere in float32,
 *       and is written to keep_prob [B,L]; otherwise keep_prob_in [B,L] is used (the strategies
 *       that sort random scores compute it between a stages == 1 and a stages == 2 call, the
 *       second reading the oracle the first wrote).
 */
int dagx_glat_glance(const int64_t *path, const int64_t *tgt_tokens, const int64_t *pred_tokens,
                     const int64_t *prev_output_tokens, const uint8_t *prev_mask, const int64_t *tgt_len,
                     const float *rand, const float *keep_prob_in, float context_p,
                     int B, int T, int L, int stages,
                     int64_t *oracle, int64_t *same_num, float *keep_prob, uint8_t *keep_mask,
                     int64_t *glat_tokens, int64_t *next_force_emit, void *stream);

/*
 * Length-penalised Viterbi decoding of the graph with on-GPU read-back and token collapsing.
 * Replaces GlatDecomposedLink.inference_viterbi (fs_plugins/models/glat_decomposed_with_link.py:720-777,
 * decode_strategy viterbi / jointviterbi) after its `.max(dim=-1)` over the vocabulary, and the
 * restore_valid_links call in front of it (:625-626): links stay in the shifted layout.
 *   links       [B,L,translen] shifted, -inf beyond out_len (as the model emits them)
 *   node_logp   [B,L] float32, node_tokens [B,L] int64: the best token of every node and its log-probability
 *   out_len     [B] int64 nodes per graph; max_length = int(2 L / decode_upsample_scale) <= 2048; L <= 1024
 *   length_penalty [max_length] float32: (t+1)^decode_viterbibeta
 *   joint != 0: jointviterbi (token log-probabilities of every node on the path count)
 * A path 0 -> x_0 -> ... -> x_{n-1} -> L_b-1 scores reach_{n-1}[x_{n-1}] + E[x_{n-1}][L_b-1] over
 * length_penalty[n-1]; among equal scores the shortest length, the lowest last node and the lowest
 * predecessors win (the first-index rule of torch.max on the host).
 *   pred_length [B] <- n;  nodes [B,max_length] <- x_k (then -1);  out_tokens [B,max_length] <- the
 *   tokens of the x_k with pads and immediate repeats dropped (the last always kept), then `pad`;
 *   out_count [B] <- how many.
 * workspace: dagx_workspace_bytes(DAGX_OP_VITERBI_DECODE, B, max_length, L, translen) bytes.
 */
int dagx_viterbi_decode(const void *links, int links_dtype, const float *node_logp, const int64_t *node_tokens,
                        const int64_t *out_len, int B, int L, int translen, int max_length,
                        const float *length_penalty, int joint, int64_t pad,
                        int64_t *out_tokens, int64_t *out_count, int64_t *pred_length, int64_t *nodes,
                        void *workspace, size_t workspace_bytes, void *stream);

/*
 * Greedy / lookahead decoding in one launch.  Replaces GlatDecomposedLink.inference_lookahead_simple
 * (fs_plugins/models/glat_decomposed_with_link.py:691-718, decode_strategy greedy / lookahead with no
 * n-gram blocking) after its `.max(dim=-1)` over the vocabulary, and the restore_valid_links call in
 * front of it (:625-626).  Arguments as dagx_viterbi_decode; L <= 4096.
 *   next(i) = argmax_j E[i][j] + node_logp[j] * beta   (greedy != 0: argmax_j E[i][j]), lowest j among equals
 *   nodes [B,L] <- 0, next(0), next(next(0)), ... up to node L_b-1 (then -1);  out_tokens [B,L] <- their
 *   tokens with pads and immediate repeats dropped (the first always kept), then `pad`;  out_count [B].
 */
int dagx_lookahead_decode(const void *links, int links_dtype, const float *node_logp, const int64_t *node_tokens,
                          const int64_t *out_len, int B, int L, int translen, float beta, int greedy, int64_t pad,
                          int64_t *out_tokens, int64_t *out_count, int64_t *nodes, void *stream);

/*
 * dagx_lsg_fwd that also returns, per row, the arg max over the vocabulary (lowest index among equal
 * logits, as torch.argmax) and the largest log-probability max(x) - lse -- in the same single pass
 * over the logits.  Replaces the extra passes of `word_ins_out.argmax(-1)` in front of the gather in
 * glat_function (fs_plugins/criterions/nat_dag_loss.py:246-250) and, with S = 0 (idx, sel and
 * their strides may then be NULL), of `output_logits.log_softmax(dim=-1)` followed by `.max(dim=-1)`
 * in decoding (fs_plugins/models/glat_decomposed_with_link.py:900, :692, :721).
 *   argmax [B*L] int64, max_logp [B*L] float32; lse may be NULL.  Logits must be free of NaN.
 */
int dagx_lsg_fwd_argmax(const void *logits, int dtype, int B, int L, int64_t V, int S,
                        const int64_t *idx, const int64_t idx_strides[3],
                        float *sel, const int64_t sel_strides[3], float *lse,
                        int64_t *argmax, float *max_logp, void *stream);

/*
 * The three operators for float64 tensors, computed in float64 throughout.  The reference instantiates its kernels
 * for double next to float and half (AT_DISPATCH_FLOATING_TYPES_AND_HALF at fs_plugins/custom_ops/dag_loss.cu:160,
 * 294, 415, 499 and dag_best_alignment.cu:150; logsoftmax_gather.cu:343-347), and the same three bound functions
 * (dag_loss.cpp:19-22, :25-28) serve them; here the float64 kernels have entry points of their own because their
 * tables are plain float64 arrays, not the residual + offset pairs of dagx_loss_fwd.  They are for checking
 * (gradcheck, a float64 run beside a float32 one), not for speed: log-domain sums, one workgroup per sweep.
 * Arguments are as for the float32 entry points unless said otherwise; all floating-point arrays are double.
 *
 * dagx_loss_f64_fwd: alpha, beta [B,T,L] contiguous (beta may be NULL when require_gradient == 0) and loss [B],
 *   alpha's read-out; rows t >= T_b and samples with invalid lengths are left unwritten (loss = -inf for those).
 * dagx_loss_f64_bwd: grad_out [B] (element stride grad_out_stride); alpha, beta, loss as written by the forward
 *   with require_gradient != 0; grad_match [B,T,L], grad_links [B,L,translen] contiguous, either may be NULL.
 * dagx_best_alignment_f64: scores are float64 with the two roundings per cell of the torch-native recurrence
 *   (fs_plugins/custom_ops/dag_loss.py:303-320), lowest index among equal predecessors (:253-257, :350).
 *   workspace: dagx_workspace_bytes(DAGX_OP_BEST_ALIGNMENT_F64, B, T, L, translen) bytes, 8-byte aligned.
 * dagx_lsg_f64_fwd / dagx_lsg_f64_bwd: as dagx_lsg_fwd / dagx_lsg_bwd with sel, grad_sel and lse double; the
 *   backward overwrites the logits with their gradient and needs lse.
 */
int dagx_loss_f64_fwd(const double *match, const int64_t match_strides[3], const double *links,
                      const int64_t *out_len, const int64_t *tgt_len, int B, int T, int L, int translen,
                      double *alpha, double *beta, double *loss, int require_gradient, void *stream);
int dagx_loss_f64_bwd(const double *grad_out, int64_t grad_out_stride, const double *alpha, const double *beta,
                      const double *loss, const double *match, const int64_t match_strides[3], const double *links,
                      const int64_t *out_len, const int64_t *tgt_len, int B, int T, int L, int translen,
                      double *grad_match, double *grad_links, void *stream);
int dagx_best_alignment_f64(const double *match, const int64_t match_strides[3], const double *links,
                            const int64_t *out_len, const int64_t *tgt_len, int B, int T, int L, int translen,
                            int64_t *path, void *workspace, size_t workspace_bytes, void *stream);
int dagx_lsg_f64_fwd(const double *logits, int B, int L, int64_t V, int S,
                     const int64_t *idx, const int64_t idx_strides[3],
                     double *sel, const int64_t sel_strides[3], double *lse, void *stream);
int dagx_lsg_f64_bwd(double *logits_inout, int B, int L, int64_t V, int S,
                     const int64_t *idx, const int64_t idx_strides[3],
                     const double *grad_sel, const int64_t gsel_strides[3], const double *lse, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DAGX_H_ */
