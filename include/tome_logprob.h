/* C ABI of libtome_logprob.so: Tome's token-log-prob path on MI355X (gfx950).
 *
 * Every entry point is a plain-C function over device pointers and sizes.  The
 * caller owns every buffer (inputs, outputs, workspace); the library never
 * allocates, frees or keeps a caller's pointer.  Launches are asynchronous on the HIP
 * stream passed as `stream` (a hipStream_t cast to void*; NULL = default
 * stream) - the caller synchronises, which mirrors MLX's lazy evaluation forced
 * by mx.eval (mlx-impl/node.py:456).  Return value: 0 on success, a negative
 * TOME_E_* code otherwise; nothing throws across this boundary.
 *
 * Conventions shared by all entry points
 *   dtype            TOME_F32 (0) or TOME_BF16 (1)
 *   targets          int32 token ids, one per row; an id outside [0, V) yields NaN
 *   row_valid        nullable int32 mask, one per row; rows with 0 are not read and
 *                    their outputs are written as 0 (argmax as -1).  It replaces the
 *                    reference's slicing by completion length (node.py:449).
 *   temperature      > 0 and finite; the reference maps 0 to 1.0 before the call
 *                    (`temperature or 1.0`, node.py:451) and so must the caller.
 *   argmax           first maximum of the row (lowest id among equal values).  The row and sampler
 *                    kernels compare the logits themselves.  The fused kernels compare the fp32 logits
 *                    they accumulate (bf16 x bf16 products summed in fp32, in the MFMA's order): the
 *                    id returned is the first maximum of THOSE numbers, so it equals the argmax of the
 *                    exact logits whenever the top two differ by more than the fp32 summation error
 *                    (about H * 2^-24 * max|h| * max|w|) and otherwise names a logit within that
 *                    error of the maximum.  NaN logits are never the maximum.
 *   out_*            float32 per row; any of out_lse / out_entropy / out_argmax may
 *                    be NULL.  lse and entropy are in nats of the temperature-scaled
 *                    logits z = x / temperature.
 *   special values   -inf logits (a masked vocabulary) carry no probability and nothing to the
 *                    entropy; a -inf target scores -inf.  A NaN logit (or hidden state) makes that
 *                    row's lse, lp and entropy NaN and leaves other rows alone.  The running maximum
 *                    starts at -1e30, the floor of the reference's kernel (mlx-impl/model.py:28): a row
 *                    whose maximum lies below it (or that holds -inf only) is outside the domain and
 *                    comes back as lse = -inf, argmax 0, lp = +inf (NaN when the target logit is -inf).
 */
#ifndef TOME_LOGPROB_H
#define TOME_LOGPROB_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TOME_ABI_VERSION 3

enum { TOME_F32 = 0, TOME_BF16 = 1 };

enum {
  TOME_OK = 0,
  TOME_E_NULL = -1,        /* a required pointer is NULL */
  TOME_E_DTYPE = -2,       /* dtype code not supported by this entry point */
  TOME_E_SHAPE = -3,       /* negative/zero/overflowing dimension or stride < V */
  TOME_E_WORKSPACE = -4,   /* workspace_bytes smaller than the *_workspace() query */
  TOME_E_TEMPERATURE = -5, /* temperature not finite or <= 0 */
  TOME_E_ALIGN = -6,       /* pointer or stride alignment the kernel needs is not met */
  TOME_E_HIP = -7,         /* a HIP runtime call failed; see tome_last_hip_error() */
  TOME_E_SCRATCH = -8      /* tome_row_logprob_noalloc: the call needs more than the fixed scratch buffer */
};

int tome_abi_version(void);
const char* tome_strerror(int code);
/* hipError_t of the last failing HIP call made by this thread inside the library (0 if none). */
int tome_last_hip_error(void);

/* ---- Row kernel: logits -> log-prob of the target id ------------------------------
 * Replaces, for one scalar per row, both
 *   local_compute_logprobs(logits, ids, temp)            mlx-impl/node.py:400-404
 *   fused_log_softmax(logits, temperature)[row, token]   mlx-impl/model.py:77-89 with the
 *                                                        host gather of node.py:571,605
 * by one single-pass online logsumexp over each row with the target gather fused in:
 *   out_lp[r] = x[r, t_r]/T - logsumexp_j(x[r, j]/T)
 * `logits` is [rows, V] with `row_stride` ELEMENTS between rows (>= V).  Rows, V and
 * strides are 64-bit: rows * V may exceed 2^31.
 */
size_t tome_row_logprob_workspace(int64_t rows, int64_t V);
int tome_row_logprob(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                     const int32_t* targets, const int32_t* row_valid, float temperature,
                     float* out_lp, float* out_lse, float* out_entropy, int32_t* out_argmax,
                     void* workspace, size_t workspace_bytes, void* stream);

/* ---- Row kernel over a list of rows -----------------------------------------------
 * The same kernel for the rows a caller names: problem i reads row row_index[i] of `logits`
 * ([n_rows, V]) and owns targets[i] and out_*[i], so inputs and outputs are PACKED in list order.
 * It replaces the reference's slicing of the completion rows out of the padded batch,
 *   chunk_logits[b, p_len - 1 : p_len - 1 + len(c_toks), :]          mlx-impl/node.py:449
 * followed by local_compute_logprobs on the slice (node.py:400-404, 451), for all sequences of a
 * chunk in one launch: prompt and padding rows are neither read nor launched, and the packed
 * result is what Completion.ref_log_probs takes (node.py:457-458).  `row_index` is a device
 * array; an entry outside [0, n_rows) is not read and scores NaN (argmax -1).  Workspace:
 * tome_row_logprob_workspace(n_index, V).
 */
int tome_row_logprob_rows(const void* logits, int dtype, int64_t n_rows, int64_t V, int64_t row_stride,
                          const int32_t* row_index, int64_t n_index, const int32_t* targets,
                          float temperature, float* out_lp, float* out_lse, float* out_entropy,
                          int32_t* out_argmax, void* workspace, size_t workspace_bytes, void* stream);

/* ---- Row kernel for callers that cannot allocate ------------------------------------
 * No counterpart in the reference.  It exists for callers that cannot hand over a workspace
 * because they cannot allocate one: code running under HIP graph capture, serving loops with
 * a fixed memory plan, harnesses that forbid hipMalloc.  Same arguments, kernels and results
 * as tome_row_logprob, minus the workspace: the per-(row, split) partials of small batches
 * go to a fixed 64 KiB array inside the library's code object (one copy per GPU, held until
 * the process ends).  The call allocates and frees nothing and, after the first call on a GPU, takes no
 * lock.  A call whose partials would not
 * fit returns TOME_E_SCRATCH before any launch (with the library's split rule - fewer than
 * 512 rows are split so that about 512 workgroups run - no shape needs more than 16 KiB).
 * All calls on one GPU share the array: calls that overlap in time on the same GPU (different
 * streams) race on it; calls on one stream, or on different GPUs, do not.  The first call on
 * each GPU looks the array's address up (hipGetSymbolAddress); make that call outside any
 * graph capture.
 */
int tome_row_logprob_noalloc(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                             const int32_t* targets, const int32_t* row_valid, float temperature,
                             float* out_lp, float* out_lse, float* out_entropy, int32_t* out_argmax,
                             void* stream);
/* Testing hook, no counterpart in the reference: lowers the number of bytes of that array a call may use
 * (0 or anything above 64 KiB restores the whole array) and returns the limit now in force, so that the
 * TOME_E_SCRATCH path, which no shape reaches with the whole array, can be exercised.  Process-wide; not for
 * production callers. */
size_t tome_row_logprob_noalloc_limit(size_t bytes);

/* ---- Decode-step sampler on the same logits pass -----------------------------------
 * Replaces, for a batch of decode rows, _sample_token(logits, temperature, top_k=20)
 * (mlx-impl/node.py:894-907) together with the log-prob lookup
 * float(fused_log_softmax(logits, T)[b, token]) (node.py:590,605 and 356,373) and the greedy
 * int(mx.argmax(logits)) (node.py:602,897):
 *   candidates   the top_k (1..32) largest logits of the row, ordered by logit descending,
 *                equal logits by ascending token id (mx.argpartition leaves ties open)
 *   out_token    uniforms == NULL: candidate 0 (the greedy token).  Otherwise the inverse CDF
 *                of softmax(candidate logits / temperature) at uniforms[row] in [0, 1): the
 *                categorical draw of node.py:906 with the randomness supplied by the caller
 *                (MLX's own random stream cannot be reproduced).
 *   out_lp       log-prob of out_token under the softmax over the WHOLE vocabulary
 *   out_argmax   first maximum of the row;  out_topk_idx / out_topk_logit  [rows, top_k], the
 *                candidates themselves (-1 / 0 past the end of a row with fewer finite logits)
 * Masked rows give token -1.  Small batches split each row over several workgroups and need
 * the workspace that tome_row_sample_workspace() sizes (0 for large batches).
 */
size_t tome_row_sample_workspace(int dtype, int64_t rows, int64_t V, int top_k);
int tome_row_sample(const void* logits, int dtype, int64_t rows, int64_t V, int64_t row_stride,
                    const float* uniforms, const int32_t* row_valid, float temperature, int top_k,
                    int32_t* out_token, float* out_lp, float* out_lse, int32_t* out_argmax,
                    int32_t* out_topk_idx, float* out_topk_logit, void* workspace,
                    size_t workspace_bytes, void* stream);

/* ---- Full log-softmax matrix ------------------------------------------------------
 * fused_log_softmax(logits, temperature) as the reference returns it
 * (mlx-impl/model.py:77-89): out[r, j] = T(x[r, j] * (1/temp)) - T(lse_r), same shape
 * and dtype as the input, the subtraction carried out in the I/O dtype (model.py:57,60).
 * `row_lse` is a caller-provided float32 buffer of `rows` elements (it receives the rows' lse);
 * workspace: tome_row_logprob_workspace(rows, V).  bf16 rows of 16384 .. 155648 elements with 16-byte aligned
 * rows are read once and written once (the row stays in one workgroup's registers), except for batches of a few dozen
 * rows or fewer when the rows are longer than 40960 elements; everything else is read twice and written once, where the
 * reference reads three times.
 */
int tome_full_log_softmax(const void* logits, void* out, int dtype, int64_t rows, int64_t V,
                          int64_t in_row_stride, int64_t out_row_stride, float temperature,
                          float* row_lse, void* workspace, size_t workspace_bytes, void* stream);

/* ---- Fused lm_head + log-softmax --------------------------------------------------
 * Replaces the pair  logits = x @ embed_tokens.weight.T  (mlx-impl/model.py:538)  +
 * local_compute_logprobs (mlx-impl/node.py:400-404) without ever writing the
 * [n_tokens, V] logits: bf16 MFMA over vocab tiles with an online logsumexp epilogue.
 *   hidden  bf16 [n_tokens, H], row stride hidden_stride elements (already normalised:
 *           the final RMSNorm of model.py:536 is the caller's)
 *   weight  bf16 [V, H] row-major (the tied embedding matrix), row stride weight_stride
 * Products are exact bf16 x bf16, accumulated in fp32; logits are NOT rounded to bf16.
 * Needs H % 8 == 0 and 16-byte aligned rows; row strides below 2^31 elements.  With H % 64 != 0
 * (the generic kernel, 32-bit byte offsets) hidden and weight must each span less than 4 GiB.
 *
 * Process-wide state of the library, all of it caches that do not change results and all of it kept per
 * device ordinal: the CU count (one workgroup per CU for batches of up to 128 tokens), a flag per large-LDS
 * kernel ("dynamic LDS limit raised", and "the 160 KB of the three-buffer sweep were refused": the two-buffer
 * sweep then serves), the device address of tome_row_logprob_noalloc's array; and the
 * two testing hooks (the selector below, tome_row_logprob_noalloc_limit).
 */
/* Testing and tuning hook, no counterpart in the reference: kind 0 / 1 makes the fused entry points take
 * the generic / LDS-DMA sweep kernel wherever its shape rules allow, 3 the LDS-DMA kernel with every vocab
 * range cut at whole 256-row tiles (no 224-row tiles, no mixed tile heights), 4 / 5 the LDS-DMA kernel with its
 * 256-token tile on two / three W buffers whatever the shape, -1 (the default, also for any other value)
 * picks by shape.  Process-wide; set it while no call of this library is running; not for
 * production callers. */
void tome_select_fused_kernel(int kind);
size_t tome_fused_lmhead_logprob_workspace(int64_t n_tokens, int64_t H, int64_t V);
int tome_fused_lmhead_logprob(const void* hidden, const void* weight, int64_t n_tokens, int64_t H,
                              int64_t V, int64_t hidden_stride, int64_t weight_stride,
                              const int32_t* targets, const int32_t* row_valid, float temperature,
                              float* out_lp, float* out_lse, float* out_entropy, int32_t* out_argmax,
                              void* workspace, size_t workspace_bytes, void* stream);

/* ---- Final RMSNorm + lm_head + log-softmax ------------------------------------------
 * The same with the model's last normalisation folded in: replaces
 *   x = self.norm(x); logits = x @ embed_tokens.weight.T      mlx-impl/model.py:536-538
 *   (RMSNorm = mx.fast.rms_norm(x, weight, eps),               mlx-impl/model.py:336-343)
 * followed by local_compute_logprobs (mlx-impl/node.py:400-404).  `hidden` holds the
 * PRE-norm states of the last decoder layer, `norm_weight` is bf16 [H].  Only rows with
 * row_valid != 0 are normalised - y = w * bf16(x * rsqrt(mean(x^2) + eps)), statistics in
 * fp32, as MLX computes it - into the workspace and then multiplied, so the prompt and pad
 * rows that node.py:443-449 computes and discards cost nothing here.
 */
size_t tome_norm_lmhead_logprob_workspace(int64_t n_tokens, int64_t H, int64_t V);
int tome_norm_lmhead_logprob(const void* hidden, const void* norm_weight, float norm_eps,
                             const void* weight, int64_t n_tokens, int64_t H, int64_t V,
                             int64_t hidden_stride, int64_t weight_stride, const int32_t* targets,
                             const int32_t* row_valid, float temperature, float* out_lp,
                             float* out_lse, float* out_entropy, int32_t* out_argmax,
                             void* workspace, size_t workspace_bytes, void* stream);

/* ---- GRPO policy + reference dual pass --------------------------------------------
 * Two lm_head weight sets over the same hidden states (policy = reference + LoRA merge,
 * mlx-impl/node.py:102-164).  Emits per token
 *   out_lp, out_ref_lp   log-probs of the target under each weight set
 *   out_k3               exp(d) - d - 1 with d = ref_lp - lp   (no counterpart in the
 *                        reference: its wire format, scheduler/proto/inference.proto:108-112,
 *                        carries only the two log-prob lists)
 *   out_entropy          entropy of the POLICY distribution (same remark)
 */
size_t tome_grpo_dual_workspace(int64_t n_tokens, int64_t H, int64_t V);
int tome_grpo_dual(const void* hidden, const void* w_policy, const void* w_ref, int64_t n_tokens,
                   int64_t H, int64_t V, int64_t hidden_stride, int64_t weight_stride,
                   const int32_t* targets, const int32_t* row_valid, float temperature,
                   float* out_lp, float* out_ref_lp, float* out_k3, float* out_entropy,
                   void* workspace, size_t workspace_bytes, void* stream);

/* ---- GRPO policy + reference pass as the reference's two models produce it ---------
 * The reference keeps two models, `self.model` (policy) and `self.reference_model`
 * (mlx-impl/node.py:65-66,443); UpdateWeights changes attention and MLP weights only
 * (node.py:134-151), so the two differ in their final HIDDEN STATES while the final norm
 * (mlx-impl/model.py:536) and the lm_head (model.py:537-538) stay shared.  This entry
 * takes one hidden-state matrix per model - both [n_tokens, H] bf16 with the same stride -
 * and one or two lm_head weights (w_ref may equal w_policy); `norm_weight` is nullable
 * and, when given, both inputs are pre-norm states as in tome_norm_lmhead_logprob.
 * Outputs as tome_grpo_dual.
 */
size_t tome_grpo_pair_workspace(int64_t n_tokens, int64_t H, int64_t V, int with_norm);
int tome_grpo_pair(const void* hidden_policy, const void* hidden_ref, const void* norm_weight,
                   float norm_eps, const void* w_policy, const void* w_ref, int64_t n_tokens,
                   int64_t H, int64_t V, int64_t hidden_stride, int64_t weight_stride,
                   const int32_t* targets, const int32_t* row_valid, float temperature,
                   float* out_lp, float* out_ref_lp, float* out_k3, float* out_entropy,
                   void* workspace, size_t workspace_bytes, void* stream);

/* ---- LoRA merge: the arithmetic of UpdateWeights -----------------------------------
 * Replaces `delta_W = scale * (lora_B @ lora_A)` (mlx-impl/node.py:128) and
 * `policy_W = base_W + delta_W` (node.py:137,146,149,151) for a batch of weight matrices in
 * one launch.  Everything is bf16; intermediates are rounded where the reference's array
 * expressions round them:  out = bf16(base + bf16(bf16(scale) * bf16(lora_B @ lora_A))),
 * the product accumulated in fp32.  A job with lora_a == NULL (and lora_b == NULL) writes
 * bf16(base + 0): the q/k/v slices the reference fills with zeros (node.py:142-145).
 * `jobs` is a HOST array, consumed before the call returns.  The workspace (device memory,
 * 16-byte aligned, size from tome_lora_merge_workspace for the same jobs) receives the job
 * table and each lora_A transposed; it must stay untouched until the launches have run.
 *   base, out     [rows, cols] bf16, strides in elements (>= cols, multiples of 8), 16-byte
 *                 aligned; out may be base itself (in place), any other overlap is undefined
 *   lora_a        [rank, cols] bf16 contiguous (LayerUpdate.lora_A, inference.proto:71)
 *   lora_b        [rows, rank] bf16 contiguous, 16-byte aligned (lora_B, inference.proto:72)
 *   rank          multiple of 8, 8..128;  cols multiple of 8
 *   scale         LayerUpdate.lora_scale; the caller maps 0 to 1.0 as node.py:127 does
 */
typedef struct TomeLoraJob {
  const void* base;
  void* out;
  const void* lora_a;
  const void* lora_b;
  int64_t rows, cols, rank, base_stride, out_stride;
  float scale;
  int32_t reserved;
} TomeLoraJob;
size_t tome_lora_merge_workspace(const TomeLoraJob* jobs, int64_t n_jobs);
int tome_lora_merge(const TomeLoraJob* jobs, int64_t n_jobs, void* workspace, size_t workspace_bytes,
                    void* stream);

/* ---- Measurement probe ---------------------------------------------------------------
 * No counterpart in the reference.  Runs the LDS -> MFMA inner loop of the fused kernel (256 x 256
 * workgroup tile, 16x16x32 bf16 MFMA, same fragment reads) on `operands` - 64 KiB of bf16 that each
 * workgroup copies into LDS once - for `steps` 64-wide K slabs: no global loads in the loop, no
 * barrier, no epilogue.  One launch does n_workgroups * steps * 2 * 256 * 256 * 64 FLOP; timing it
 * with random operands gives the bf16 MFMA rate this part sustains under its power limit, which
 * bench.py reports beside the published peak.  flags & 1: every wave also issues the fused kernel's
 * eight 1 KiB global -> LDS requests per slab (re-reading `operands`, which stays in the caches): the
 * cost of the fill apart from the L2 side.  flags & 2: after every 16 slabs (one vocab tile at
 * K = 1024; `steps` is rounded down to a multiple) the accumulators are folded with the arithmetic of
 * the fused kernel's online-softmax epilogue.  flags & 4: the fused kernel's workgroup barrier in
 * every step.  All three together are that kernel at H = 1024 on a memory system that always answers
 * from cache.  `operands` must hold at least 64 KiB (`operand_bytes`) and `sink` receives
 * n_workgroups * 512 floats (`sink_bytes` must cover them); smaller buffers, n_workgroups outside
 * 1..4096, steps outside 1..65536 and flags outside 0..7 return TOME_E_SHAPE before any launch (one
 * launch is at most a few hundred milliseconds of GPU time).
 */
int tome_probe_mfma_ceiling(const void* operands, size_t operand_bytes, int n_workgroups, int steps,
                            int flags, float* sink, size_t sink_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* TOME_LOGPROB_H */
