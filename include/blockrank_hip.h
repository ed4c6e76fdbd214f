/* C ABI of libblockrank_hip.so: BlockRank block-sparse prefill attention and attention-score
 * ranking on one MI355X (gfx950).
 *
 * The reference (nilesh2797/BlockRank) has no native layer; its path is entered through two Hugging
 * Face registries (src/blockrank/blockrank_std_attention.py:652-665,
 * src/blockrank/blockrank_triton_kernel_attention.py:938-965).  Each entry point below names the
 * reference function whose work it takes over.  All pointers are device pointers unless stated;
 * all strides are in elements; `stream` is a hipStream_t passed as void*.  Calls enqueue work on
 * the stream and return without synchronising.  Return value 0 = success; anything else = failure,
 * with the reason available from br_last_error() on the calling thread.
 *
 * Layout vocabulary: a batch of B sequences, each M blocks of H token slots (S = M*H).  Block 0 is
 * the instruction prefix, blocks 1..M-2 the documents, block M-1 the query.  Inside a block the real
 * tokens form one contiguous span (left padding puts it at the end of the block).
 */
#ifndef BLOCKRANK_HIP_H
#define BLOCKRANK_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BR_DTYPE_F32 0
#define BR_DTYPE_BF16 1
#define BR_DTYPE_F16 2  /* forward attention, scores, rotary embedding; no backward, no fp8 variant, no log-sum-exp output */

#define BR_OK 0
#define BR_ERR_ARG 1      /* bad shape, dtype, alignment or null pointer (reference: AssertionError) */
#define BR_ERR_SPACE 2    /* a caller-provided buffer is too small */
#define BR_ERR_HIP 3      /* a HIP runtime call or launch failed */
#define BR_ERR_PLAN 4     /* br_plan_check: the plan's launch counters are not at rest */

/* Library version, major*10000 + minor*100 + patch. */
int br_version(void);

/* Message for the last failure on this thread ("" if none). */
const char* br_last_error(void);

/* Tokens per query tile the kernels use for this head layout (the plan depends on it). 0 if the
 * layout is unsupported (Nq not a multiple of Nkv). */
int br_tile_tokens(int Nq, int Nkv);

/* Size, in int32 elements, of the plan buffer for a (B, M, H) batch with this head layout. */
size_t br_plan_ints(int B, int M, int H, int Nq, int Nkv);

/* A plan carries the ticket counters of the persistent attention kernel; the last workgroup of every launch puts them
 * back to zero.  A launch that did not run to its end (a fault, a killed process sharing the buffer) leaves them
 * counting, and the next launch on that plan would hand out no work.  br_plan_check waits for `stream`, reads the
 * counters back and returns BR_OK or BR_ERR_PLAN (the only entry point that synchronises: for diagnostics, not for
 * the serving path); br_plan_rearm enqueues their reset (a small kernel: safe under graph capture).  No reference
 * counterpart: its mask tensor has no state. */
int br_plan_check(const int32_t* plan, void* stream);
int br_plan_rearm(int32_t* plan, void* stream);

/* Build the request plan (block table + work items) from the (B, M, H) block mask, one byte per
 * token slot, non-zero = real token.  Replaces eager_blockrank_attention_mask /
 * triton_blockrank_attention_mask (blockrank_std_attention.py:264-309,
 * blockrank_triton_kernel_attention.py:887-935): the 5-D additive mask those build carries exactly
 * the per-block real-token spans, which is all the kernels need.  Build once per forward pass and
 * pass to every layer.  One plan must not be used by two streams at the same time. */
int br_plan_build(const uint8_t* valid, int B, int M, int H, int Nq, int Nkv, int32_t* plan, size_t plan_ints,
                  void* stream);

/* Same, from per-block real-token counts (B*M int32 on the device) instead of a mask; left_padded
 * says at which end of its H slots each block's span sits.  No reference counterpart: it is the
 * entry for callers that never build the padded mask
 * (block layout of block_icr_collate_fn, src/blockrank/dataset.py:219-227). */
int br_plan_build_from_lengths(const int32_t* lens, int left_padded, int B, int M, int H, int Nq, int Nkv,
                               int32_t* plan, size_t plan_ints, void* stream);

/* Plan for a PACKED token layout: the real tokens of all blocks of all sequences follow each other on
 * the token axis with no padded slots (sequence 0 block 0, block 1, ..., sequence 1 block 0, ...), so
 * q, k, v and out are (1, heads, T, D) / (1, T, heads, D) tensors with T = sum of lens and the calls
 * below take batch strides of 0.  lens: B*M int32 real-token counts on the device; H: an upper bound
 * of the block lengths (it sizes the plan and defines the row positions of the score calls: position
 * H-1 is a block's last token).  Same B, M, H go to every later call.  No reference counterpart: the
 * reference pads every block to a common H (src/blockrank/dataset.py:205-227); this is the layout of
 * a collate function that does not. */
int br_plan_build_packed(const int32_t* lens, int B, int M, int H, int Nq, int Nkv, int32_t* plan, size_t plan_ints,
                         void* stream);

/* Bytes of scratch br_prefill_fwd needs: the split-KV partials of the query blocks' key walks.  The plan cuts those
 * walks only as far as it takes to give every workgroup of the grid work, and takes the slots from one pool for the
 * whole batch, so the size follows from the head layout and the current device's compute-unit count and does not grow
 * with B (about 18 MB for 32 / 8 heads of dim 128 on 256 compute units).  0 without a HIP device. */
size_t br_prefill_workspace_bytes(int B, int Nq, int Nkv, int D);

/* Block-sparse prefill attention.  Replaces sdpa_blockrank_attention_forward /
 * eager_blockrank_attention_forward (blockrank_std_attention.py:472-650, :96-262) and
 * triton_blockrank_attention_forward (blockrank_triton_kernel_attention.py:798-884) including their
 * repeat_kv expansion and final transpose copy.
 *   q (B, Nq, S, D), k and v (B, Nkv, S, D), out (B, Nq, S, D) logical shapes; *_strides give the
 *   element strides of (batch, head, token); the head dimension must be dense, every stride a
 *   multiple of 16 bytes, every base pointer 16-byte aligned.  out as the reference returns it,
 *   (B, S, Nq, D) contiguous, is strides {S*Nq*D, D, Nq*D}.
 *   Rows of real tokens receive the attention output; rows of padded slots are set to zero.
 *   D in {64, 128}; dtype BR_DTYPE_BF16 or BR_DTYPE_F16 (MFMA of that type, fp32 softmax/accumulate) or BR_DTYPE_F32. */
int br_prefill_fwd(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq,
                   int Nkv, int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides,
                   const int64_t* v_strides, const int64_t* out_strides, float scale, int dtype, void* workspace,
                   size_t workspace_bytes, void* stream);

/* br_prefill_fwd that also records two hipEvent_t (either may be NULL) on the stream immediately
 * before and after the main attention kernel, so a caller can time that kernel alone inside a longer
 * sequence of work.  No reference counterpart (the reference has no timing hooks). */
int br_prefill_fwd_events(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq,
                          int Nkv, int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides,
                          const int64_t* v_strides, const int64_t* out_strides, float scale, int dtype,
                          void* workspace, size_t workspace_bytes, void* stream, void* ev_start, void* ev_stop);

/* br_prefill_fwd for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and
 * result as br_prefill_fwd without the workspace: the split-KV partials live in a device array that
 * belongs to the library (br_prefill_noalloc_max_workspace_bytes() = 32 MiB on every GPU the library is
 * used on, until the process ends).  Neither this call nor anything it calls allocates or frees memory: the
 * array's address on a device is looked up by the br_plan_build* calls (the first of them on a device loads the
 * library's code object, which is when the runtime sets the array up), and every request needs a plan, so by the
 * time this entry runs - under graph capture too - the address is known.
 * A request whose br_prefill_workspace_bytes() exceeds that size is refused with BR_ERR_SPACE (no head layout
 * of a current model does: 32 / 8 heads of dim 128 need about 18 MB whatever the batch).  Every call on a GPU
 * uses that GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream,
 * one after the other, do not.  Nothing in the array has to be cleared between calls (a call reads only the
 * partials it wrote itself). */
size_t br_prefill_noalloc_max_workspace_bytes(void);
int br_prefill_fwd_noalloc(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq,
                           int Nkv, int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides,
                           const int64_t* v_strides, const int64_t* out_strides, float scale, int dtype, void* stream);

/* Bytes of the score-partials buffer of br_prefill_fwd_scores. */
size_t br_score_partials_bytes(int B, int Nq, int M, int H, int score_rows);

/* br_prefill_fwd_events that, in the same pass, leaves what the per-document scores of the query
 * block's last score_rows positions (H-score_rows .. H-1) need: for every head, such row and
 * earlier-block key tile the pair (max, sum of exp) of the row's logits over the tile, in score_part.
 * This is the reference's "attention + s_last in one call" (blockrank_std_attention.py:623-645;
 * triton_blockrank_attention_forward with return_last_block_scores,
 * blockrank_triton_kernel_attention.py:858-881) without the second pass over K; the reference uses
 * score_rows = 16.  bf16 and fp16 (BR_DTYPE_F32 callers use br_doc_scores).  score_part needs no
 * initialisation; it is consumed by br_doc_scores_from_partials with the same plan. */
int br_prefill_fwd_scores(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq,
                          int Nkv, int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides,
                          const int64_t* v_strides, const int64_t* out_strides, float scale, int dtype,
                          void* workspace, size_t workspace_bytes, int score_rows, float* score_part,
                          size_t score_part_bytes, void* stream, void* ev_start, void* ev_stop);

/* Everything optional about a forward call in one structure, for br_prefill_fwd_ex.  Zero-initialise it, set
 * struct_bytes = sizeof(BrPrefillOptions) and fill in what the call should do; members left zero / NULL switch
 * their feature off.
 *   ev_start, ev_stop   hipEvent_t recorded around the main kernel, as in br_prefill_fwd_events.
 *   score_part, score_part_bytes, score_rows
 *                       the score partials of br_prefill_fwd_scores (bf16).
 *   fp8_tokens          > 0: the fp8 Q K^T variant of br_prefill_fwd_fp8qk; the workspace is then sized by
 *                       br_prefill_fp8qk_workspace_bytes.
 *   lse, lse_strides    the log-sum-exp output of br_prefill_fwd_lse (bf16, no fp8).
 *   rope_cos, rope_sin, rope_strides
 *                       the rotary position embedding of Q inside the attention kernel (bf16, no fp8): q holds the
 *                       query projection's output as it is, cos and sin are the tables (batch or 1, tokens, D) of the
 *                       model's rotary module on q's token axis (rope_strides: element strides of batch and token,
 *                       multiples of 8; a batch stride of 0 is one table for all sequences), and every Q row is rotated
 *                       in registers when the kernel loads it: x cos + rotate_half(x) sin in fp32, rounded once, as
 *                       br_rope_qk computes it.  K must come rotated (br_rope_qk with Nq = 0 does K alone).  Replaces
 *                       the Q half of apply_rotary_pos_emb in the Hugging Face model files (transformers
 *                       models/mistral/modeling_mistral.py, the same in llama and qwen2), which the reference reaches
 *                       through the model forward of scripts/eval_attn.py:139-151.
 *   rank_rows, rank_R, rank_scale, rank_scores
 *                       with score_part: the per-document scores of br_doc_scores_from_partials(score_part, plan,
 *                       rank_rows, rank_R, score_rows, ..., out_scale = rank_scale, scores = rank_scores, probs = NULL)
 *                       for a caller that knows the rows to score before the layer runs (the reference finds them
 *                       from the labels, losses.py:43-48, which do not depend on the forward): the reduction runs in the
 *                       first workgroups of the launch that merges the split partials, so the whole call is two launches.
 *                       rank_rows (B, rank_R) int32 and rank_scores (B, M-2) fp32 on the device. */
typedef struct BrPrefillOptions {
    size_t struct_bytes;
    void* ev_start;
    void* ev_stop;
    float* score_part;
    size_t score_part_bytes;
    int32_t score_rows;
    int32_t rank_R;
    int64_t fp8_tokens;
    float* lse;
    const int64_t* lse_strides;
    const void* rope_cos;
    const void* rope_sin;
    const int64_t* rope_strides;
    const int32_t* rank_rows;
    float* rank_scores;
    float rank_scale;
} BrPrefillOptions;

/* br_prefill_fwd with the options above (opt may be NULL: then it is br_prefill_fwd).  Same checks and error codes as
 * the single-purpose entry points, which are this call with one feature set. */
int br_prefill_fwd_ex(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv,
                      int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                      const int64_t* out_strides, float scale, int dtype, void* workspace, size_t workspace_bytes,
                      const BrPrefillOptions* opt, void* stream);

/* Bytes of scratch br_prefill_fwd_fp8qk needs: the split-KV partials plus the quantised K, the per-block maxima
 * (B*M*Nkv) and the scales.  tokens: length of the token axis summed over the batch (B*M*H for the padded layout,
 * the number of real tokens for a packed one). */
size_t br_prefill_fp8qk_workspace_bytes(int B, int Nq, int Nkv, int D, int M, int64_t tokens);

/* br_prefill_fwd_scores with the Q K^T products of the prefix and document blocks computed in fp8 e4m3
 * and P V in bf16.  q, k, v, out are bf16 as in br_prefill_fwd.  K is first quantised per (sequence, kv
 * head) with the power-of-two scale 2^(floor(log2(max|x|)) - 7), the maximum taken over the real tokens
 * (x / scale rounded to e4m3, written into the workspace); Q is converted by the attention kernel itself,
 * in registers, every query row with the scale its own maximum gives by the same rule (a power of two
 * makes the division exact); the products run on the fp8 matrix cores and the scales are folded into the
 * softmax scale.  The query block's rows - the ones the per-document scores are read from - are computed
 * on the bf16 Q and K, so the score partials are those of br_prefill_fwd_scores.  D = 128 only.
 * score_part may be NULL (then score_rows is ignored).  No reference counterpart: the reference computes
 * Q K^T in the model dtype (blockrank_std_attention.py:549-620); this is the reduced-precision variant
 * for Qwen2.5-shaped ranking whose scores must stay within 5e-3 relative of the fp32 result with the
 * same top-10. */
int br_prefill_fwd_fp8qk(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq,
                         int Nkv, int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides,
                         const int64_t* v_strides, const int64_t* out_strides, float scale, int64_t tokens,
                         void* workspace, size_t workspace_bytes, int score_rows, float* score_part,
                         size_t score_part_bytes, void* stream, void* ev_start, void* ev_stop);

/* Per-document relevance from the partials of br_prefill_fwd_scores: compute_auxiliary_attention_loss(
 * answer_ids=None, return_logits=True) (src/blockrank/losses.py:37-78).
 *   rows: (B, R) int32 indices 0..score_rows-1 into the last score_rows positions of the query block
 *   (what losses.py:43-48 computes from the labels); R <= 16.  scores, probs, out_scale as in
 *   br_doc_scores. */
int br_doc_scores_from_partials(const float* score_part, const int32_t* plan, const int32_t* rows, int R,
                                int score_rows, int B, int Nq, int M, int H, float out_scale, float* scores,
                                float* probs, void* stream);

/* Bytes of scratch br_doc_scores needs. */
size_t br_doc_scores_workspace_bytes(int B, int Nq, int M, int R);

/* Fused per-document relevance.  Replaces the pair "raw logits of the last rows"
 * (blockrank_std_attention.py:623-645; compute_last_block_attention_scores,
 * blockrank_triton_kernel_attention.py:542-606) + compute_auxiliary_attention_loss(answer_ids=None,
 * return_logits=True) (src/blockrank/losses.py:37-78) without materialising the logits.
 *   rows: (B, R) int32, positions 0..H-1 inside the query block of the rows to use (the reference
 *   uses the "[" token and the one before it); R <= 16.
 *   scores: (B, M-2) fp32 = out_scale * sum over heads and rows of the document's probability mass
 *   under a softmax of scale*q.k over all real document tokens.  The reference's mean over heads and
 *   rows divided by the temperature is out_scale = 1 / (Nq * R * temperature).
 *   probs: optional (B, Nq, R, M-2) fp32 per-head, per-row document probabilities, or NULL.
 *   Of q only the rows named by `rows` are read (tokens (M-1)*H + rows[b][r]), so a caller that has
 *   projected the query block alone may pass a base pointer shifted accordingly. */
int br_doc_scores(const void* q, const void* k, const int32_t* plan, const int32_t* rows, int R, int B, int Nq,
                  int Nkv, int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, float scale,
                  float out_scale, int dtype, float* scores, float* probs, void* workspace, size_t workspace_bytes,
                  void* stream);

/* The reference's s_last tensor itself, for callers that consume it directly: logits (B, Nq, R, S)
 * fp32 = scale * q.k + (0 where the row may see the key, else neg), for the rows given as in
 * br_doc_scores.  Replaces blockrank_std_attention.py:242-262 / :639-645 and
 * _compute_last_block_scores_kernel (blockrank_triton_kernel_attention.py:432-535).  neg is the
 * reference's 0.7 * finfo(dtype).min. */
int br_last_block_logits(const void* q, const void* k, const int32_t* plan, const int32_t* rows, int R, int B,
                         int Nq, int Nkv, int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides,
                         float scale, float neg, int dtype, float* logits, void* stream);

/* Gradient of br_last_block_logits with respect to q and k, given the gradient of its output: what torch autograd
 * derives for the s_last tensor of the reference's trainable hooks (blockrank_std_attention.py:242-262, :639-645), through
 * which the auxiliary attention loss trains (trainer.py:91-101, losses.py:53-74).
 *   dlogits (B, Nq, R, M*H) fp32.  Real rows against real keys carry gradient (also keys the row may not see: the mask is
 *   an added constant); slots without a token and rows that are padding carry none, as in br_last_block_logits.
 *   dq: a zero-filled tensor addressed like q (element strides dq_strides); only the R chosen rows of every head are
 *   written (rows named twice are summed).  dk: addressed like k (dk_strides); every key token is written (in the padded
 *   layout the empty slots get zero), so it needs no initialisation.  dtype of q, k, dq, dk: 0 fp32, 1 bf16.
 *   Padded and packed layouts; R <= 16 per call. */
int br_last_block_logits_bwd(const float* dlogits, const void* q, const void* k, const int32_t* plan, const int32_t* rows, int R, int B,
                             int Nq, int Nkv, int M, int H, int D, const int64_t* q_strides, const int64_t* k_strides, float scale,
                             int dtype, void* dq, const int64_t* dq_strides, void* dk, const int64_t* dk_strides, void* stream);

/* Rotary position embedding of Q and K in one pass, the step in front of every attention call:
 * out = x * cos + rotate_half(x) * sin, rotate_half(x) = (-x[D/2:], x[:D/2]).  Replaces apply_rotary_pos_emb of
 * the Hugging Face model the reference ranks with (transformers models/mistral/modeling_mistral.py,
 * rotate_half and apply_rotary_pos_emb; the same function in the Llama and Qwen2 model files), which the
 * reference reaches through the model forward of scripts/eval_attn.py:139-151 and scripts/train.py.
 *   q (B, Nq, S, D), k (B, Nkv, S, D) logical, element strides (batch, head, token) as for br_prefill_fwd;
 *   cos, sin (B, S, D) with element strides (batch, token) - a batch stride of 0 broadcasts one table;
 *   q_out (B, S, Nq, D), k_out (B, S, Nkv, D) contiguous: the layout whose head-transposed views the
 *   attention entry points take.  dtype 0 fp32, 1 bf16 for all six tensors; D 64 or 128.
 *   Nq = 0 rotates K alone (q, q_out and q_strides are then ignored and may be NULL): the step that goes with
 *   the rope_cos / rope_sin option of br_prefill_fwd_ex, which rotates Q itself.
 * fp32 arithmetic with one rounding of the result (the reference's eager bf16 expression rounds every
 * intermediate product and the sum). */
int br_rope_qk(const void* q, const void* k, const void* cos, const void* sin, void* q_out, void* k_out, int B, int Nq, int Nkv, int S,
               int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* cs_strides, int dtype, void* stream);

/* ---- training: forward that also saves the log-sum-exp, and the backward ----
 * The reference trains through its torch hooks ("default_blockrank" and relatives,
 * blockrank_std_attention.py:96-262 and :472-650, called by the aux-loss trainer, trainer.py:79-101), which
 * torch autograd differentiates; its Triton hook raises NotImplementedError on backward
 * (blockrank_triton_kernel_attention.py:759-761).  These two entry points are the hand-written counterpart.
 *
 * br_prefill_fwd_lse: br_prefill_fwd for bf16 tensors that also writes, for every real query token,
 *   lse[b * lse_strides[0] + head * lse_strides[1] + token] = log2( sum over visible keys of 2^(scale*log2(e)*q.k) )
 * (the natural log-sum-exp is lse * ln 2).  token is the index on the token axis of q (m*H + position for the
 * padded layout, the running token index for a packed one, whose lse_strides[0] is 0).  Padded slots are not written.
 */
int br_prefill_fwd_lse(const void* q, const void* k, const void* v, void* out, const int32_t* plan, int B, int Nq, int Nkv, int M,
                       int H, int D, const int64_t* q_strides, const int64_t* k_strides, const int64_t* v_strides,
                       const int64_t* out_strides, float scale, void* workspace, size_t workspace_bytes, float* lse,
                       const int64_t* lse_strides, void* stream);

/* Bytes of scratch br_prefill_bwd needs (fp32 dQ sums of the query block's rows, dK and dV sums of the prefix keys, and
 * rowsum(dO * O) per row and head).  token_slots = B*M*H for the padded layout, the packed token count otherwise. */
size_t br_prefill_bwd_workspace_bytes(int B, int Nq, int Nkv, int H, int D, int64_t token_slots);

/* Gradients of the attention output with respect to q, k and v (bf16, D 64 or 128):
 *   P = softmax(scale * q.k over visible keys),  dV = P^T dO,  dS = P * (dO V^T - rowsum(dO * O)),
 *   dQ = scale * dS K,  dK = scale * dS^T Q,  dK and dV summed over the query heads of a kv head.
 * q, k, v, out, lse and plan exactly as given to / written by br_prefill_fwd_lse, with lse dense:
 * lse_strides = (Nq*M*H, M*H) for the padded layout, (0, token_slots) for a packed one.  dout has out's logical
 * shape (B, Nq, S, D) with its own strides; dq (B, Nq, S, D), dk, dv (B, Nkv, S, D) with their strides.  Rows of
 * padded slots receive zeros; dout on padded slots is ignored.  Sums with one owner are kept in registers in a
 * fixed order; dQ of a query block whose key walk is split over several workgroups and dK, dV of the prefix keys
 * (one workgroup per viewing block) are summed with fp32 atomic adds, so their last bits depend on the order in
 * which the workgroups finish. */
int br_prefill_bwd(const void* q, const void* k, const void* v, const void* out, const void* dout, const float* lse,
                   const int32_t* plan, int B, int Nq, int Nkv, int M, int H, int D, const int64_t* q_strides,
                   const int64_t* k_strides, const int64_t* v_strides, const int64_t* out_strides, const int64_t* dout_strides,
                   const int64_t* lse_strides, void* dq, void* dk, void* dv, const int64_t* dq_strides, const int64_t* dk_strides,
                   const int64_t* dv_strides, float scale, int64_t token_slots, void* workspace, size_t workspace_bytes,
                   void* stream);

/* ---- the elementwise steps of a decoder layer around the attention, one pass each ----
 * Both replace methods of the Hugging Face model classes the reference's models are instances of (transformers
 * models/mistral/modeling_mistral.py: MistralRMSNorm.forward, MistralMLP.forward; the same in the Llama and Qwen2
 * model files), which the ranking forward of scripts/eval_attn.py:139-151 runs in every decoder layer.
 *
 * br_rmsnorm: out[r, :] = weight * (x[r, :] * rsqrt(mean(x[r, :]^2) + eps)), fp32 arithmetic; for bf16 the normalised
 * value is rounded to bf16 before the multiplication by the weight, as in the model file.  x, out: rows x hidden with
 * the given row strides (elements); weight: hidden.  dtype 0 fp32, 1 bf16.
 * br_silu_mul: out = silu(gate) * up over n contiguous elements (silu rounded to the tensor type first). */
int br_rmsnorm(const void* x, const void* weight, void* out, int64_t rows, int hidden, int64_t x_row_stride, int64_t out_row_stride,
               float eps, int dtype, void* stream);
int br_silu_mul(const void* gate, const void* up, void* out, int64_t n, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BLOCKRANK_HIP_H */
