/*
 * axon_amd.h — C ABI of libaxon_amd.so (gfx950 / MI355X).
 *
 * The reference (modelcorp/axon) is pure Python and has no FFI; its plugin
 * points for this path are Python callables.  Every entry point below is the
 * device-side body of one of those callables and cites the reference function
 * it stands behind.  The Python mirror in axon_amd/ binds them with ctypes.
 *
 * Conventions
 *  - plain pointers to DEVICE memory, int64 sizes, scalars by value, an opaque
 *    hipStream_t passed as void*;
 *  - return 0 on success, a negative AXON_ERR_* code otherwise; never throws,
 *    never exits, never synchronises, never allocates (the one exception is
 *    documented at the function);
 *  - workspace is caller-provided; *_workspace_bytes() gives the size;
 *  - all launches go to `stream`; results are valid once that stream reaches
 *    the point after the call.
 *  - "rows": stage-2/3 kernels address a flat array of n_slots values split
 *    into n_rows rows by int32 offsets cu_seqlens[n_rows+1].  The reference's
 *    padded [B,T] layout is the special case cu_seqlens = {0,T,2T,...}; pass
 *    uniform_len=T then (cu_seqlens may be NULL), else uniform_len=0.
 */
#ifndef AXON_AMD_H
#define AXON_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AXON_AMD_ABI_VERSION 20

enum {
  AXON_OK = 0,
  AXON_ERR_ARG = -1,       /* null pointer / bad enum / bad scalar            */
  AXON_ERR_SHAPE = -2,     /* size constraint violated (see each function)    */
  AXON_ERR_WORKSPACE = -3, /* workspace too small or misaligned               */
  AXON_ERR_LAUNCH = -4,    /* hipGetLastError() after a launch was not success */
  AXON_ERR_DEVICE = -5,    /* not a gfx950 device                             */
  AXON_ERR_TOO_LARGE = -6  /* beyond the fixed capacity of a no-allocation entry point */
};

/* mask element types accepted by stage-2/3 kernels (response_mask is int64 in
 * the reference's production pipeline, float in its unit tests). */
enum { AXON_MASK_F32 = 0, AXON_MASK_I64 = 1 };

int axon_amd_abi_version(void);
const char* axon_amd_error_string(int code);

/* ------------------------------------------------------------------------- *
 * (a) LM head: log-prob + entropy without materialising [tokens x vocab]
 * ------------------------------------------------------------------------- */

/* Forward.  Replaces efficient_entropy_forward
 * (axon/utils/kernel/kernels.py:506-695) as called by LinearCrossEntropy.forward
 * (axon/utils/kernel/linear_cross_entropy.py:50-99) with reduction "none", and
 * _fused_linear_for_ppo_fwd (axon/utils/torch/fused_linear.py:26-46) evaluated
 * with fp32 accumulation.
 *   hidden  [n_tokens, hidden] bf16 row-major, 16-byte aligned rows
 *   weight  [vocab, hidden]    bf16 row-major
 *   labels  [n_tokens] int32 or int64; ids outside [0,vocab) contribute logit 0
 *   out: logprobs, entropy [n_tokens] fp32;
 *        lse = logsumexp(logits/T), entropy_b = sum softmax*logits/T  [n_tokens]
 *        fp32, the statistics the backward needs (the reference saves
 *        maximum/accumulate/entropy_b, linear_cross_entropy.py:93).
 *   softcap > 0 applies Gemma-style logit soft-capping, logits = softcap *
 *        tanh(logits / softcap), before the temperature
 *        (_apply_logit_softcapping, axon/utils/torch/fused_linear.py:19-23;
 *        the reference's Triton kernels have no such option and its models fall
 *        back to the torch path, axon/models/transformers/dense_common.py:201-219);
 *        0 = none.  Pass the same value to the backward.
 *   seq_start (may be NULL): token-aligned packed layout.  `labels` is then the
 *        packed stream of token ids itself and seq_start[p] = 1 where a sequence
 *        begins (axon_seq_start_flags).  Hidden position n predicts the token at
 *        n + 1: the label is labels[n + 1] and logprobs / entropy are written at
 *        n + 1; sequence starts receive 0.  This is torch.roll(ids, -1) before the
 *        head (axon/utils/fsdp/forward_utils.py:131) and the shift-right after it
 *        (rmpad_postprocess, forward_utils.py:164-182) folded into the kernels.
 *        lse / entropy_b stay indexed by hidden position.  The backward takes the
 *        same flags and reads dlogprobs / dentropy in the aligned layout, ignoring
 *        them at sequence starts.
 *   stash (may be NULL): device memory of axon_lmhead_stash_bytes bytes, 16-byte aligned, that
 *        the forward fills for its backward: every softmax numerator as fp16, relative to the
 *        maximum of its 128-row part of the vocabulary (2 bytes per logit, in tile order), and
 *        those maxima.  A backward given the same buffer reads the dlogits off it instead of
 *        recomputing the logits: 6 N H V flop per forward + backward instead of 8, for
 *        2 * n_tokens * vocab bytes that must live from the forward to the backward (10 GB at
 *        32768 x 151936; the part has 288 GB).  The reference keeps no such buffer (its kernels
 *        recompute, kernels.py:1377-1585; its torch path keeps the fp32 logits of one chunk,
 *        fused_linear.py:26-46).  fp16 holds eleven bits of each numerator whatever the size of
 *        the logit; numerators below 2^-24 of their part's maximum read back as 0.
 * Constraints: hidden % 32 == 0, hidden >= 32, vocab >= 1, n_tokens >= 0. */
int64_t axon_lmhead_fwd_workspace_bytes(int64_t n_tokens, int64_t hidden, int64_t vocab);
/* Bytes of the forward's stash for this shape; 0 if the shape cannot be stashed (tiles that are
 * shifted back inside the matrix need n_tokens % 4 == 0 and vocab % 4 == 0), -1 for an invalid
 * shape.  The layout is private to the library and depends on the shape only. */
int64_t axon_lmhead_stash_bytes(int64_t n_tokens, int64_t hidden, int64_t vocab);
/* flags[p] = 1 where a non-empty sequence of cu_seqlens[n_seqs + 1] begins, else 0.
 * `flags` holds n_tokens bytes rounded up to a multiple of 4. */
int axon_seq_start_flags(const int32_t* cu_seqlens, int64_t n_seqs, int64_t n_tokens,
                         uint8_t* flags, void* stream);
int axon_lmhead_fwd(const void* hidden_bf16, const void* weight_bf16, const void* labels,
                    int labels_are_i64, int64_t n_tokens, int64_t hidden, int64_t vocab,
                    float inv_temperature, float softcap, const uint8_t* seq_start,
                    float* logprobs, float* entropy, float* lse,
                    float* entropy_b, void* workspace, int64_t workspace_bytes, void* stash,
                    int64_t stash_bytes, void* stream);

/* Backward.  Replaces efficient_entropy_backward
 * (axon/utils/kernel/kernels.py:1377-1585, default _Split_Dlogits_N) and
 * _fused_linear_for_ppo_bwd (axon/utils/torch/fused_linear.py:49-89):
 *   dlogit = [g*(onehot - p) - gH*p*(logit/T - entropy_b)] / T, rounded to bf16,
 *   d_hidden = dlogit @ W, d_weight = dlogit^T @ hidden, both written as bf16.
 * With softcap > 0 dlogit is additionally multiplied by 1 - tanh^2(raw logit / softcap)
 * (fused_linear.py:80-83).  dentropy may be NULL (treated as zeros).  vocab_chunk (multiple of 256, or 0
 * for the library default, 32768) bounds the bf16 dlogit scratch to
 * 2 * n_tokens_padded * vocab_chunk * 2 bytes.  stash (may be NULL): what axon_lmhead_fwd left
 * for the same operands, shape, temperature and softcap; the dlogits are then decoded from it by
 * a streaming kernel (2 bytes read, 4 written per logit) and the logits are not recomputed. */
int64_t axon_lmhead_bwd_workspace_bytes(int64_t n_tokens, int64_t hidden, int64_t vocab,
                                        int64_t vocab_chunk);
int axon_lmhead_bwd(const float* dlogprobs, const float* dentropy, const void* hidden_bf16,
                    const void* weight_bf16, const void* labels, int labels_are_i64,
                    const float* lse, const float* entropy_b, int64_t n_tokens, int64_t hidden,
                    int64_t vocab, float inv_temperature, float softcap,
                    const uint8_t* seq_start, void* d_hidden_bf16, void* d_weight_bf16,
                    int64_t vocab_chunk, void* workspace, int64_t workspace_bytes,
                    const void* stash, int64_t stash_bytes, void* stream);

/* Rows of the backward without an upstream gradient.  The reference's trainer runs the head over every
 * packed token, prompt included (fsdp_model_forward, axon/utils/fsdp/forward_utils.py:236-265), and the
 * loss weighs every token with response_mask, which is zero on the prompt (agg_loss,
 * axon/trainer/algos/loss/utils.py:120-251): the dlogprobs / dentropy of those positions arrive as exact
 * zeros, and so do those of tokens that the correction rejects or the loss clips.  Such a row's dlogit is zero: it adds nothing to d_weight and
 * its d_hidden row is zero (efficient_entropy_backward, axon/utils/kernel/kernels.py:1377-1585,
 * computes them all the same).  These three calls let the host run axon_lmhead_bwd over the other
 * rows only.
 *   axon_lmhead_active_rows: row_index[r] = the r-th hidden row (ascending) whose dlogprobs or
 *        dentropy is not zero (NaN counts as not zero); with seq_start both are read at the aligned
 *        position n + 1 and sequence starts never count.  row_rank[n] = r for such a row, -1 for the
 *        others; count[0] = their number.  row_index and row_rank hold n_tokens entries.  One
 *        workgroup; the numbering is the same on every run.
 *   axon_lmhead_gather_rows: the operands of those rows, compact: hidden_c[r] = hidden[row_index[r]],
 *        lse_c, entropy_b_c likewise; labels_c (same integer type as labels), dlogprobs_c, dentropy_c
 *        (may be NULL; zeros where dentropy is NULL) from the aligned position.  They are operands of
 *        axon_lmhead_bwd with n_tokens = n_active and seq_start = NULL.
 *   axon_lmhead_scatter_rows: d_hidden[n] = d_hidden_c[row_rank[n]], or zeros where row_rank[n] < 0.
 * hidden % 8 == 0; hidden, hidden_c, d_hidden, d_hidden_c on 16-byte boundaries. */
int axon_lmhead_active_rows(const float* dlogprobs, const float* dentropy, const uint8_t* seq_start,
                            int64_t n_tokens, int32_t* row_index, int32_t* row_rank, int32_t* count,
                            void* stream);
int axon_lmhead_gather_rows(const void* hidden_bf16, const void* labels, int labels_are_i64,
                            const float* lse, const float* entropy_b, const float* dlogprobs,
                            const float* dentropy, const uint8_t* seq_start, int64_t n_tokens,
                            int64_t hidden, const int32_t* row_index, int64_t n_active,
                            void* hidden_c_bf16, void* labels_c, float* lse_c, float* entropy_b_c,
                            float* dlogprobs_c, float* dentropy_c, void* stream);
int axon_lmhead_scatter_rows(const void* d_hidden_c_bf16, const int32_t* row_rank, int64_t n_tokens,
                             int64_t hidden, void* d_hidden_bf16, void* stream);

/* Timed variants for benchmarks: same work, plus HIP events recorded on `stream`
 * around every launch into a timer object.  Recording does not synchronise;
 * axon_timer_collect synchronises the timer's stream, ADDS the elapsed milliseconds
 * and launch counts of everything recorded since the last collect to the two HOST
 * arrays of 8 entries (zero them first) and forgets the spans:
 *   [0] forward logits+statistics kernel, [1] merge, [2] label logit, [3] unused,
 *   [4] backward transposes, [5] dlogit (recompute, or decode of the stash), [6] dHidden GEMM, [7] dWeight GEMM.
 * The timer creates and destroys events and owns host memory (the exception to
 * "never allocates"); `stream` of a timed call must be the timer's.
 * No reference counterpart (measurement only). */
void* axon_timer_create(void* stream); /* NULL on failure */
int axon_timer_collect(void* timer, float* phase_ms, int32_t* phase_launches);
void axon_timer_destroy(void* timer);
int axon_lmhead_fwd_timed(const void* hidden_bf16, const void* weight_bf16, const void* labels,
                          int labels_are_i64, int64_t n_tokens, int64_t hidden, int64_t vocab,
                          float inv_temperature, float softcap, const uint8_t* seq_start,
                          float* logprobs, float* entropy, float* lse, float* entropy_b,
                          void* workspace, int64_t workspace_bytes, void* stash,
                          int64_t stash_bytes, void* stream, void* timer);
int axon_lmhead_bwd_timed(const float* dlogprobs, const float* dentropy, const void* hidden_bf16,
                          const void* weight_bf16, const void* labels, int labels_are_i64,
                          const float* lse, const float* entropy_b, int64_t n_tokens, int64_t hidden,
                          int64_t vocab, float inv_temperature, float softcap,
                          const uint8_t* seq_start, void* d_hidden_bf16, void* d_weight_bf16,
                          int64_t vocab_chunk, void* workspace, int64_t workspace_bytes,
                          const void* stash, int64_t stash_bytes, void* stream, void* timer);

/* One step as token blocks.  The reference's per-micro-batch step (CausalLM.forward_backward_fn,
 * axon/models/fsdp_models.py:183-279) runs the head forward over all tokens, then the loss, then the
 * head backward; its kernels hold [tokens, 9504]-column slices of logits on the way
 * (efficient_entropy_forward / _backward, axon/utils/kernel/kernels.py:1523-1580).  These entry
 * points run the same three stages block of consecutive tokens by block: forward of the block over the whole
 * vocabulary with a stash (axon_lmhead_fwd above), the caller's loss kernels on the block's positions,
 * backward of the block from the stash, then the next block.  What lives from a forward to its
 * backward is ONE block's stash (2 bytes x block tokens x vocab), whatever the number of tokens, and
 * the path executes 6 N H V flop for the 6 that count.  All calls of a step go to one stream.
 *   Arrays: `hidden`, `labels`, `seq_start`, `logprobs`, `entropy`, `dlogprobs`, `dentropy`, `d_hidden`
 *        point at the BLOCK's first position inside the step's whole arrays (hidden rows and d_hidden
 *        rows of the block; the per-position arrays offset by the block's first position); `lse`,
 *        `entropy_b` are per block (n_tokens entries).  `weight`, `d_weight`, `dw_acc` are whole.
 *   last_dst (token-aligned layout only, seq_start != NULL): a block's last row predicts the position
 *        after the block: pass n_tokens when the stream goes on (its label, outputs and gradients are
 *        then read and written at index n_tokens of the block-offset arrays, i.e. the next block's
 *        first position), and minus the block's first position when the block ends the stream (index 0
 *        of the whole arrays, a sequence start).  0 is the whole-stream call, as axon_lmhead_fwd.
 *   axon_lmhead_block_begin: once per step, before the first backward: the transposed weight into
 *        `workspace` (the same workspace, of axon_lmhead_bwd_workspace_bytes(largest block, ...) bytes,
 *        must then be handed to every axon_lmhead_block_bwd of the step, with wt_ready = 1).  For
 *        hidden >= 256 and vocab % 64 == 0 the backward reads the weight where it lies: the call then
 *        launches nothing and the workspace holds no transposed weight.
 *   axon_lmhead_block_bwd: d_hidden rows of the block (bf16, complete: a row sums over the vocabulary
 *        only).  The weight gradient sums over all blocks: dw_mode 0 = this block is the whole step,
 *        d_weight (bf16) is written; 1 = first block, dw_acc (fp32 partial sums,
 *        axon_lmhead_block_dw_acc_bytes(hidden, vocab) bytes, 16-byte aligned; its layout is private:
 *        tile by tile in register order, so that it streams at full width) is written;
 *        2 = a middle block, added to dw_acc; 3 = last block, dw_acc + this block's share is rounded
 *        to bf16 into d_weight and dw_acc is left as it was.  The same vocab_chunk in every call of a
 *        step.  stash may be NULL (the block's logits are then recomputed).
 *   timer: NULL, or an axon_timer_create object on `stream` (phases as below).
 * axon_scale_bf16_unless_one multiplies n bf16 values in place by the DEVICE scalar scale[0] and touches
 * nothing when it is exactly 1 (the step's gradients are finished before autograd hands over the
 * factor of the loss, which is 1 unless the caller scaled the loss); n % 8 == 0, x on a 16-byte boundary. */
int64_t axon_lmhead_block_dw_acc_bytes(int64_t hidden, int64_t vocab);
int axon_lmhead_block_begin(const void* weight_bf16, int64_t hidden, int64_t vocab, int64_t vocab_chunk,
                            void* workspace, int64_t workspace_bytes, void* stream, void* timer);
int axon_lmhead_block_fwd(const void* hidden_bf16, const void* weight_bf16, const void* labels,
                          int labels_are_i64, int64_t n_tokens, int64_t hidden, int64_t vocab,
                          float inv_temperature, float softcap, const uint8_t* seq_start,
                          int64_t last_dst, float* logprobs, float* entropy, float* lse,
                          float* entropy_b, void* workspace, int64_t workspace_bytes, void* stash,
                          int64_t stash_bytes, void* stream, void* timer);
int axon_lmhead_block_bwd(const float* dlogprobs, const float* dentropy, const void* hidden_bf16,
                          const void* weight_bf16, const void* labels, int labels_are_i64,
                          const float* lse, const float* entropy_b, int64_t n_tokens, int64_t hidden,
                          int64_t vocab, float inv_temperature, float softcap,
                          const uint8_t* seq_start, int64_t last_dst, void* d_hidden_bf16,
                          void* d_weight_bf16, float* dw_acc, int dw_mode, int wt_ready,
                          int64_t group_pos, int dw_now, int64_t ws_tokens,
                          int64_t vocab_chunk, void* workspace, int64_t workspace_bytes,
                          const void* stash, int64_t stash_bytes, void* stream, void* timer);
int axon_lmhead_block_can_group(int64_t hidden, int64_t vocab, int64_t vocab_chunk);
/* How many bf16 copies of a chunk's dlogits the backward (axon_lmhead_bwd, axon_lmhead_block_bwd) writes for
 * this shape: 1 = token-major only (the weight-gradient GEMM reads it K-major), 2 = token-major and
 * vocab-major (hidden < 256, vocab % 8 != 0, or a last vocabulary chunk of fewer than 256 rows).  For
 * byte accounting; negative for an unsupported shape.  No reference counterpart. */
int axon_lmhead_bwd_dlogit_copies(int64_t hidden, int64_t vocab, int64_t vocab_chunk);
int axon_scale_bf16_unless_one(void* x_bf16, int64_t n, const float* scale, void* stream);

/* Plain bf16 NT GEMM on the same MFMA main loop, out[n][m] = sum_k A[m][k]*B[n][k]
 * (fp32 accumulate, fp32 output).  No reference counterpart: it exists so tests
 * and the benchmark can measure the main loop in isolation.
 * Constraints: k % 32 == 0, lda/ldb multiples of 8 elements. */
int axon_gemm_nt_bf16(const void* a_bf16, int64_t lda, const void* b_bf16, int64_t ldb,
                      float* out, int64_t ldo, int64_t m, int64_t n, int64_t k, void* stream);

/* The same GEMM with either operand given K-MAJOR instead of K-contiguous: a_kmajor != 0 means `a` is
 * [k][lda] with the m rows contiguous (out[n][m] = sum_k a[k][m] * b[n][k]), likewise b_kmajor for `b`.
 * A K-major operand is read as it lies (no transposed copy) through the LDS transpose read of gfx950.
 * No reference counterpart (test and benchmark helper, like the above).  K-major operands only on the
 * DMA main loop: m, n >= 256, k % 64 == 0, and for a K-major operand a 16-byte aligned base and a row
 * count and leading dimension that are multiples of 8; AXON_ERR_SHAPE otherwise. */
int axon_gemm_bf16(const void* a_bf16, int64_t lda, int a_kmajor, const void* b_bf16, int64_t ldb,
                   int b_kmajor, float* out, int64_t ldo, int64_t m, int64_t n, int64_t k, void* stream);

/* ------------------------------------------------------------------------- *
 * (b) ragged segmented reductions over cu_seqlens
 * ------------------------------------------------------------------------- */

/* Per-row statistics in one pass over the tokens:
 *   cnt[r]  = sum_t mask                      (mask NULL -> 1)
 *   sum[r]  = sum_t (a - b) * mask            (b NULL -> 0)
 *   flag[r] = any_t  mask != 0 && cond(a-b)   cond: flag_mode 1: (a-b) <  flag_threshold
 *                                                   flag_mode 2: |a-b| > flag_threshold
 *                                                   flag_mode 0: no flag (flag may be NULL)
 * Any of cnt/sum/flag may be NULL.  cnt and flag must be zero-filled by the caller
 * (axon_fill_zero); sum needs no initialisation but a zero-filled, 8-byte aligned sum_workspace of
 * axon_row_stats_workspace_bytes(n_rows) bytes: the partial sums of a row that spans several
 * wavefronts are added there as 64-bit fixed-point integers (units of 2^-32; partials of 2^20 or more
 * in magnitude and non-finite ones in a float beside), so sum[r] repeats bit for bit from run to run
 * whatever the row lengths, like the reference's CPU sums (axon/utils/rl/sampler.py:70-83), and a
 * second small launch writes sum[].  Serves masked row sums in
 * compute_sampler_rejection_mask (axon/utils/rl/sampler.py:70-79), the veto
 * any() (sampler.py:418-420), GSPO's sequence mean (axon/trainer/algos/loss/loss.py:143-145),
 * agg_loss row counts (axon/trainer/algos/loss/utils.py:236-251), GRPO's score sum
 * (axon/trainer/algos/advantages/advantage.py:98) and the zero-advantage row test
 * (axon/utils/rl/utils.py:35-36). */
int64_t axon_row_stats_workspace_bytes(int64_t n_rows);
int axon_row_stats(const float* a, const float* b, const void* mask, int mask_kind,
                   const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots, int64_t uniform_len,
                   int flag_mode, float flag_threshold, float* cnt, float* sum, int32_t* flag,
                   void* sum_workspace, void* stream);

/* group_mean_std (axon/utils/rl/advantage.py:106-150) + the GRPO scalar
 * (axon/trainer/algos/advantages/advantage.py:98-107):
 *   count/s1/s2 by group, mean, var with Bessel, std = sqrt(max(var, eps)),
 *   count<=1 -> mean 0, std 1;
 *   norm_by_std 1 / 0: scalar[i] = (score[i]-mean[g])/(std[g]+eps) or score-mean; * (count[g] > 1);
 *   norm_by_std 2: RLOO / LOOP (advantage.py:112-146): (n*s - S_g)/(n-1), 0 for singleton groups;
 *   norm_by_std 3: GPG (advantage.py:336-371): rows/count_nonzero(scores) * (s - mean[g]) / eps,
 *                  with eps carrying f_norm.
 * mean/std/count [n_groups] are outputs AND scratch: zero-fill them first.
 * scalar may be NULL (plain group_mean_std).  Single workgroup; n_rows < 2^31. */
int axon_group_stats(const float* scores, const int64_t* gidx, int64_t n_rows, int64_t n_groups,
                     float eps, int norm_by_std, float* mean, float* std, float* count,
                     float* scalar, void* stream);

/* out[t] = row_scalar[row(t)] * mask[t]  — `scalars.unsqueeze(-1) * response_mask`
 * (axon/trainer/algos/advantages/advantage.py:108). clamp_abs > 0 applies
 * compute_advantage's optional clamp (advantages/__init__.py:73-74). */
int axon_row_broadcast_mask(const float* row_scalar, const void* mask, int mask_kind,
                            const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots,
                            int64_t uniform_len, float clamp_abs, float* out, void* stream);

/* ------------------------------------------------------------------------- *
 * (c) elementwise kernels
 * ------------------------------------------------------------------------- */

int axon_fill_zero(void* ptr, int64_t n_bytes, void* stream); /* n_bytes % 4 == 0 */
/* out[i] = x[i] * s1[0] * s2[0] (s2 may be NULL: 1), the scalars read on the device: the backward of the loss
 * operators, whose forward leaves the per-token gradient without the upstream factor and, for a token-mean whose
 * denominator is known only at the end of the pass, without acc[5] (torch.autograd's multiply in the reference,
 * e.g. the backward of agg_loss, axon/trainer/algos/loss/utils.py:120-187).  x and out on 16-byte boundaries
 * (out may be x). */
int axon_scale_f32(const float* x, const float* s1, const float* s2, float* out, int64_t n, void* stream);

/* Bytes of the `partials` workspace of axon_sampler_correction / axon_policy_loss /
 * axon_side_terms / axon_cov_policy_loss / axon_gmpo_loss (the same for every n_slots: 8 floats for
 * each of at most 16384 workgroups that walk the tokens, 8 floats for each group of 64 workgroups,
 * then 2 KB of ticket counters).  The scalar sums of those kernels (the reference's masked_mean
 * metrics and agg_loss totals, axon/utils/torch/ops.py:131-145,
 * axon/trainer/algos/loss/utils.py:224-251) are added from per-workgroup partials in a fixed order
 * inside the same launch (the workgroup that finishes last in a group adds the group, the one that
 * finishes last of all adds the groups), so results are reproducible run to run and no same-address
 * float atomics are involved.
 * The ticket counters (the last 2048 bytes) must be ZERO before the first use; every launch leaves
 * them zero again, so one zero-filled workspace serves any number of calls that are ordered on a
 * stream.  Two launches that overlap in time must not share a workspace.  The rows need no
 * initialisation. */
int64_t axon_reduce_partials_bytes(int64_t n_slots);

/* Sampler/trainer correction, compute_sampler_correction_and_rejection_mask
 * (axon/utils/rl/sampler.py:334-446).  lr = old - sampler.
 *   is_mode: 0 off, 1 token, 2 sequence        (sampler.py:206-231)
 *   rs_mode: 0 off, 1 token, 2 sequence, 3 geometric   (sampler.py:66-83)
 *   veto: has_veto != 0, log_veto = fp32 log(threshold) computed by the caller
 *   rs_lr_lo / rs_lr_hi: the closed log-space interval equivalent to
 *       lower <= exp(clamp(lr,-20,20)) <= upper in fp32, computed by the caller;
 * row_cnt,row_sum,row_flag: outputs of axon_row_stats(old, sampler, mask, flag_mode 1,
 * log_veto); may be NULL when neither a row-level mode nor the veto is on.
 * Outputs: is_weights [n_slots] (NULL if is_mode 0), new_mask [n_slots] fp32 =
 * mask * rs * veto.  acc[8] (written, not accumulated; untouched when n_slots == 0)
 * receives sums for the metrics: [0] sum mask,
 * [1] sum is_w(before truncation)*mask, [2] sum (1-rs)*mask, [3] sum catastrophic*mask,
 * [4] rows vetoed, [5] sum truncated is_w * mask.
 * partials: workspace of axon_reduce_partials_bytes(n_slots). */
int axon_sampler_correction(const float* old_logp, const float* sampler_logp, const void* mask,
                            int mask_kind, const int32_t* cu_seqlens, int64_t n_rows,
                            int64_t n_slots, int64_t uniform_len, int is_mode, float is_threshold,
                            int rs_mode, float rs_lr_lo, float rs_lr_hi, int has_veto,
                            float log_veto, const float* row_cnt, const float* row_sum,
                            const int32_t* row_flag, float* is_weights, float* new_mask,
                            float* acc, float* partials, void* stream);

/* Diagnostics of the sampler / trainer mismatch in one token pass and one row pass, for a single
 * host readback.  Replaces the ~60 separate reductions (each with its own .item()) of
 * _compute_is_metrics / _compute_rs_metrics (axon/utils/rl/sampler.py:106-173, 259-326),
 * compute_offpolicy_metrics (sampler.py:454-518) and compute_trainer_sampler_mismatch_metrics
 * (axon/utils/metrics/trainer_sampler_mismatch_metrics.py:36-80).
 *   lr = old - sampler, e = exp(clamp(lr, -20, 20)), pa = exp(old), ps = exp(sampler); every
 *   quantity is taken over tokens with mask != 0.
 *   is_mode / rs_mode as in axon_sampler_correction; is_lo/is_hi, rs_lo/rs_hi: ratio thresholds
 *   (lower, upper) in fp32; rs_lr_lo/rs_lr_hi: the log-space interval of the token-level rejection
 *   (same values as passed to axon_sampler_correction); log_*: fp32 log of the ratio thresholds.
 *   workspace: axon_sampler_diag_workspace_bytes(n_rows, n_slots) bytes, 8-byte aligned, whose
 *   first 6 * n_rows floats the caller has zero-filled.
 * out[72] (double):
 *   sums   [0] mask  [1] e  [2] e^2  [3] lr  [4] exp(lr)-lr-1  [5] e>is_hi  [6] e<is_lo
 *          [7] clamp(e,is)  [8] clamp(e,is)^2  [9] e>rs_hi  [10] e<rs_lo  [11] clamp(e,rs)
 *          [12] clamp(e,rs)^2  [13] |pa-ps|  [14] |pa-ps|^2  [15] |lr|  [16] lr^2  [17] pa  [18] ps
 *          [19] pa^2  [20] ps^2  [21] pa*ps  [22] token-level rejected
 *   rows   x = masked row mean of the untruncated weight:
 *          [23..26] IS: sum x, sum x^2, #x>is_hi, #x<is_lo      [27..30] RS: the same
 *          row-level modes, L = row log-ratio (sum, or masked mean for geometric), w = exp(clamp L):
 *          [31..35] IS: #L>log_is_hi, #L<log_is_lo, sum w*cnt, sum clamp(w)*cnt, sum clamp(w)^2*cnt
 *          [36..40] RS: the same   [41] rows rejected (token mode: rows with a rejected valid token)
 *          a, b = masked row means of old / sampler:  [42] sum exp(-a)  [43] sum -a  [44] sum exp(-b)
 *          [45] sum -b  [46] sum (b-a)  [47] sum |b-a|  [48] sum exp(b-a)  [49] sum exp(2 clamp(sum lr))
 *   maxima [50] e  [51] |pa-ps|  [52] |lr|  [53] IS x  [54] IS |x-1|  [55] RS x  [56] RS |x-1|
 *          [57] IS L  [58] RS L  [59] b-a          minima [60..69]: the same slots ([64],[66] unused) */
int64_t axon_sampler_diag_workspace_bytes(int64_t n_rows, int64_t n_slots);
int axon_sampler_diag(const float* old_logp, const float* sampler_logp, const void* mask, int mask_kind,
                      const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots, int64_t uniform_len,
                      int is_mode, float is_lo, float is_hi, int rs_mode, float rs_lo, float rs_hi,
                      float rs_lr_lo, float rs_lr_hi, float log_is_lo, float log_is_hi,
                      float log_rs_lo, float log_rs_hi, float* workspace, double* out, void* stream);

/* Per-row weights of agg_loss (axon/trainer/algos/loss/utils.py:120-251) folded
 * into one multiplier per row, plus GSPO's per-row mean log-ratio:
 *   token_reduce: 0 sum, 1 mean, 2 mean-norm, 3 mean-program
 *   batch_reduce: 0 token-mean, 1 step-mean, 2 program-mean
 *   row_cnt/row_sum from axon_row_stats(logp, old, mask).
 *   per_row_token_count / num_program_tokens / num_program_steps: optional
 *   double [n_rows] (counts as floating values, as the reference divides by them,
 *   utils.py:224-229: a fractional count is not truncated);
 *   valid_count: optional double pointer whose element [0] is
 *   the mini-batch-wide denominator (utils.py:224-229), else computed locally.
 * Outputs row_scale[n_rows], row_mean[n_rows] (= row_sum / max(row_cnt,1)).
 * Up to 64 workgroups: each repeats the pass over the counts (same order, same totals) and writes its share of the rows. */
int axon_loss_row_scale(const float* row_cnt, const float* row_sum, int64_t n_rows,
                        int64_t row_len_for_norm, int token_reduce, int batch_reduce,
                        const double* per_row_token_count, const double* num_program_tokens,
                        const double* num_program_steps, const double* valid_count,
                        float* row_scale, float* row_mean, void* stream);

/* Clipped policy loss, forward and gradient in one pass.
 *   kind 0: ppo_loss_fn  (axon/trainer/algos/loss/loss.py:47-111), dual clip c
 *   kind 1: gspo_loss_fn (axon/trainer/algos/loss/loss.py:114-180)
 *   kind 2: reinforce_loss_fn / gpg_loss_fn (loss.py:183-197, 471-512): -A * logp * is_weights
 *   kind 3: cispo_loss_fn (loss.py:411-468): -sg(clamp(ratio)) * A * logp; clip_c != 0 switches
 *           the optional token-level mask on; is_weights must be NULL
 *   kind 4: value_loss_fn (loss.py:547-591) without its factor 0.5: logp carries vpreds, old_logp the
 *           old values, adv the returns, ratio_lo the cliprange_value; max((vpreds - returns)^2,
 *           (clip_by_value(vpreds, values -+ cliprange) - returns)^2) with torch's tie rules for the
 *           gradient; acc[1] = sum mask*(clipped term larger), acc[2] = sum mask*vpreds
 * ratio_lo / ratio_hi: the clamp bounds 1 - clip_ratio_low and 1 + clip_ratio_high,
 * evaluated in double by the caller and rounded to fp32 (what torch.clamp does
 * with Python scalars).  clip_c: dual-clip constant (> 1), PPO only.
 * row_scale: per-row multiplier from axon_loss_row_scale, or NULL with
 * uniform_scale applied to every token.
 * post_normalize != 0 (row_scale NULL, any kind but 1): `sum` / `token-mean`
 * aggregation in ONE pass over the tokens (utils.py:224-229): the kernel sums
 * uniform_scale * loss * mask, then divides the total by max(valid_count[0], 1), or by
 * max(sum mask, 1) when valid_count is NULL; grad[] is left WITHOUT that division and
 * acc[5] returns the factor 1/denominator the caller multiplies the gradient by
 * (it multiplies by the upstream gradient anyway).  Otherwise acc[5] = 1.
 * Outputs grad[n_slots] = d loss / d log_probs and acc[8] (written, not
 * accumulated; untouched when n_slots == 0): [0] loss,
 * [1] sum mask*(pg2>pg1), [2] sum mask*(-(logp-old)), [3] sum mask*((c1>pg3)&(A<0)),
 * [4] sum mask, [5] gradient factor.
 * partials: workspace of axon_reduce_partials_bytes(n_slots). */
int axon_policy_loss(int kind, const float* logp, const float* old_logp, const float* adv,
                     const void* mask, int mask_kind, const float* is_weights,
                     const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots,
                     int64_t uniform_len, const float* row_scale, const float* row_mean,
                     float uniform_scale, int post_normalize, const double* valid_count,
                     float ratio_lo, float ratio_hi, float clip_c, float* grad, float* acc,
                     float* partials, void* stream);

/* The policy losses that need a per-row quantity, in ONE pass over the tokens: GSPO's sequence mean
 * log-ratio (axon/trainer/algos/loss/loss.py:141-151) and every aggregation of agg_loss with a per-row
 * divisor (token_reduce mean / mean-norm / mean-program, batch_reduce step-mean / program-mean,
 * axon/trainer/algos/loss/utils.py:120-251).  Replaces axon_row_stats + axon_loss_row_scale +
 * axon_policy_loss for those cases (which read log_probs, old_log_probs and the mask twice): a
 * workgroup owns whole rows, keeps their tokens in registers between the row sums and the token
 * pass, and forms the row sums in a fixed order without atomics, so the sequence ratio repeats bit
 * for bit from run to run.  A row of more than 2048 tokens is read a second time, all but its last
 * 2048.  A workgroup works on one row (or two short ones) at a time, so the kernel suits batches
 * whose rows are at least some tens of tokens long on average (for shorter rows use the calls it
 * replaces).
 *   kind, masks, ratio_lo / ratio_hi / clip_c, grad, acc[0..5]: as in axon_policy_loss (kinds 0-4).
 *   token_reduce / batch_reduce / per_row_token_count / num_program_tokens / num_program_steps /
 *   valid_count: as in axon_loss_row_scale.  Without valid_count the batch denominator (sum of the
 *   mask for token-mean, number of rows with a mask token for step-mean) is known only at the end:
 *   acc[0] is divided by it, grad[] is left WITHOUT that division and acc[5] returns the factor the
 *   caller multiplies the gradient by; with valid_count acc[5] = 1.
 *   Slots that belong to no row (before cu_seqlens[0], after cu_seqlens[n_rows]) receive grad 0.
 *   n_slots of 1, 2 or 3 is refused (AXON_ERR_SHAPE): the kernel reads 16-byte vectors; such inputs are
 *   for the calls it replaces.  The same holds for axon_sampler_correction_rows.
 *   The per-token arrays (logp, old_logp, adv, mask, is_weights, grad; in axon_sampler_correction_rows
 *   old_logp, sampler_logp, mask, is_weights, new_mask) must start on 16-byte boundaries (AXON_ERR_ARG
 *   otherwise): every multiple of four slots is then a 16-byte vector.  cu_seqlens must be non-decreasing
 *   with 0 <= cu_seqlens[r] <= n_slots (not checked on the device: a row that runs backwards or past the
 *   arrays would be read out of bounds).
 * partials: workspace of axon_reduce_partials_bytes, ticket counters zero (see there). */
int axon_policy_loss_rows(int kind, const float* logp, const float* old_logp, const float* adv,
                          const void* mask, int mask_kind, const float* is_weights,
                          const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots,
                          int64_t uniform_len, int token_reduce, int batch_reduce,
                          const double* per_row_token_count, const double* num_program_tokens,
                          const double* num_program_steps, const double* valid_count, float ratio_lo,
                          float ratio_hi, float clip_c, float* grad, float* acc, float* partials,
                          void* stream);

/* axon_sampler_correction for the modes that need a per-row quantity (the per-sequence veto,
 * sampler.py:413-428; sequence-level weights :210-214; sequence / geometric rejection :70-79), in ONE
 * pass over the tokens, same scheme as axon_policy_loss_rows: 20 bytes per token instead of 32, and
 * row sums formed in a fixed order, so a row whose sum sits next to a rejection bound takes the same
 * side on every run.  Arguments as axon_sampler_correction without the row inputs; row_cnt /
 * row_sum / row_flag (each may be NULL) receive the per-row sum of the mask, of (old - sampler) *
 * mask and the veto decision.  acc as in axon_sampler_correction. */
int axon_sampler_correction_rows(const float* old_logp, const float* sampler_logp, const void* mask,
                                 int mask_kind, const int32_t* cu_seqlens, int64_t n_rows,
                                 int64_t n_slots, int64_t uniform_len, int is_mode, float is_threshold,
                                 int rs_mode, float rs_lr_lo, float rs_lr_hi, int has_veto,
                                 float log_veto, float* is_weights, float* new_mask, float* row_cnt,
                                 float* row_sum, int32_t* row_flag, float* acc, float* partials,
                                 void* stream);

/* axon_policy_loss for callers that cannot allocate.  No counterpart in the reference: it is
 * for code under HIP graph capture, tight serving loops and harnesses that forbid
 * hipMalloc, which cannot obtain the `partials` workspace.  Arguments, outputs and results
 * are those of axon_policy_loss (same kernels) without `partials`: the per-workgroup partial
 * sums and the ticket counters go to a fixed 522 KB array in device memory that the library holds on every GPU it
 * runs on until the process ends.  Calls no hipMalloc / hipFree and no allocating routine.
 *   n_slots <= 16 777 216 (2^24 tokens, the capacity this entry point states and is tested
 *   for); larger inputs return AXON_ERR_TOO_LARGE and launch nothing.
 * The first call on a device looks the array's address up (hipGetSymbolAddress, with that
 * device current) and must therefore happen outside stream capture; later calls on that
 * device only launch.  All calls on one GPU share the array: calls that overlap in time on
 * one GPU (different streams) race on it; calls ordered on one stream, or by events, do not.
 * The array's ticket counter starts at zero (static storage) and every launch leaves it zero, the
 * partial sums are overwritten before they are read: nothing is cleared between calls. */
int axon_policy_loss_noalloc(int kind, const float* logp, const float* old_logp, const float* adv,
                             const void* mask, int mask_kind, const float* is_weights,
                             const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots,
                             int64_t uniform_len, const float* row_scale, const float* row_mean,
                             float uniform_scale, int post_normalize, const double* valid_count,
                             float ratio_lo, float ratio_hi, float clip_c, float* grad, float* acc,
                             void* stream);

/* The non-fused branch of fsdp_model_forward (axon/utils/fsdp/forward_utils.py:287-304): the model has
 * written logits [n, vocab] (row stride ld elements; dtype AXON_LOGITS_F32 or AXON_LOGITS_BF16, already
 * divided by the temperature).  One read of each row gives
 *   logprob[t] = log_softmax(logits[t])[labels[t]]    (logprobs_from_logits, axon/utils/torch/ops.py:39-102)
 *   entropy[t] = logsumexp(logits[t]) - sum softmax*logits   (entropy_from_logits, ops.py:105-120)
 *   lse[t]     = logsumexp(logits[t])                 (kept for the backward)
 * in fp32.  logprob (with labels) or entropy may be NULL.  A label outside [0, vocab) gives logprob 0. */
enum { AXON_LOGITS_F32 = 0, AXON_LOGITS_BF16 = 1 };
int axon_logits_fwd(const void* logits, int dtype, int64_t ld, int64_t n, int64_t vocab,
                    const void* labels, int labels_are_i64, float* logprob, float* entropy, float* lse,
                    void* stream);

/* Backward of the above in one read and one write of the rows:
 *   dlogits[t][j] = g_logprob[t] (onehot - p) - g_entropy[t] p (log p + entropy[t]),  p = exp(logits - lse)
 * in the logits' dtype.  g_logprob or g_entropy may be NULL (that output had no gradient).  dlogits may be
 * the logits' own storage (the in-place backward of the reference's flash-attn cross entropy,
 * ops.py:70-75, inplace_backward). */
int axon_logits_bwd(const void* logits, int dtype, int64_t ld, int64_t n, int64_t vocab,
                    const void* labels, int labels_are_i64, const float* lse, const float* entropy,
                    const float* g_logprob, const float* g_entropy, void* dlogits, int64_t ld_dlogits,
                    void* stream);

/* KL penalty inside the reward, the tensor part of apply_kl_penalty (axon/utils/rl/kl.py:276-322):
 *   kld = kl_penalty(old_logp, ref_logp, kl_type) * mask      (types as in axon_kl_penalty)
 *   rewards = scores - beta * kld
 *   row_vals[0][r] = sum_t mask,  row_vals[1][r] = sum_t kld  (row_vals [2][n_rows], zero-filled by the caller)
 * from which the caller forms current_kl = mean_r(row_vals[1][r] / max(row_vals[0][r], 1)) for its KL
 * controller. */
int axon_kl_reward(const float* scores, const float* old_logp, const float* ref_logp, const void* mask,
                   int mask_kind, const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots,
                   int64_t uniform_len, int kl_type, float beta, float* rewards, float* row_vals,
                   void* stream);

/* Time recurrences of the return-based advantage estimators, run from each row's last token to its
 * first (axon/trainer/algos/advantages/advantage.py), before any whitening:
 *   mode 0: gae_advantage_fn :57-73.  nextvalues and lastgaelam skip tokens with mask 0 (a fractional
 *           mask blends as in the reference); adv = lastgaelam, ret = adv + values.
 *   mode 1: chunked_gae_advantage_fn :480-537 (_chunked_gae_core :374-477): the same recurrence over the
 *           tokens with mask > 0 only, V past the last response token = 0; adv = ret = 0 elsewhere.
 *   mode 2: reinforce_plus_plus_advantage_fn :163-171: ret[t] = r[t] + gamma * mask[t+1] * ret[t+1];
 *           adv is not written (may be NULL).
 *   mode 3: remax_advantage_fn :234-238: ret[t] = sum_{s>=t} r[s]*mask[s];
 *           adv = ret - row_baseline[row] * mask.
 * values is read by modes 0 and 1, lam by modes 0 and 1, row_baseline [n_rows] by mode 3.
 * Rows as in axon_row_stats (uniform_len > 0: padded [n_rows, uniform_len]; else cu_seqlens). */
int axon_reverse_scan(int mode, const float* rewards, const float* values, const void* mask,
                      int mask_kind, const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots,
                      int64_t uniform_len, float gamma, float lam, const float* row_baseline,
                      float* adv, float* ret, void* stream);

/* masked_whiten (axon/utils/rl/advantage.py:153-190): mean and variance over the mask (variance times
 * n/(n-1) when n > 1), out = (x - mean) * rsqrt(var + 1e-8), times the mask when remask != 0 (the
 * `* response_mask` of advantage.py:174,215).  out may equal x, or be NULL for the statistics alone.
 * stats[4] (device): mean, n, variance, rsqrt(variance + 1e-8).  partials: workspace of
 * axon_masked_whiten_workspace_bytes(n_slots) bytes; the sums are formed in a fixed order.
 * x, mask and out 16-byte aligned. */
int64_t axon_masked_whiten_workspace_bytes(int64_t n_slots);
int axon_masked_whiten(const float* x, const void* mask, int mask_kind, int64_t n_slots, int remask,
                       float* out, float* stats, float* partials, void* stream);

/* Per-row scalars of the group-based estimators that need more than a group mean and deviation
 * (advantage.py).  The caller passes the groups in compressed form: members[n_rows] = row indices ordered
 * by group (row order kept within a group), offsets[n_groups + 1] into members.
 *   mode 0: opo_advantage_fn :260-277: score - (n > 1 ? sum(len*score)/max(sum len, 1) : 0)
 *   mode 1: reinforce_plus_plus_baseline_advantage_fn :197-210: score - (n > 1 ? group mean : 0)
 *   mode 2: grpo_passk_advantage_fn :304-330: the best row of a group gets max - second max, divided by
 *           (unbiased std + eps) when normalize != 0; every other row 0 (groups of one row: the caller
 *           raises before the launch, as the reference does)
 *   mode 3: kimi_k1_5_advantage_fn :586-623: score + length term (coef = the scheduled length_coef,
 *           threshold = correct_threshold, min/max length over the whole group, off when coef <= 0),
 *           then (shaped - mean)/(std + eps) or shaped - mean, 0 for groups of one row
 * lens [n_rows] (sum of the response mask per row) is read by modes 0 and 3. */
int axon_group_scalar(int mode, const float* scores, const float* lens, const int32_t* members,
                      const int32_t* offsets, int64_t n_rows, int64_t n_groups, float eps,
                      int normalize, float coef, float threshold, float* scalar, void* stream);

/* Token selection of the covariance-based losses (axon/trainer/algos/loss/loss.py):
 *   kind 0: kl_cov_loss_fn :311-330.  Over the tokens with mask > 0: covariance
 *           (A - mean A) * (logp - mean logp) with plain means; the k = max(1, int(count * ratio)) largest
 *           are selected (torch.topk there).
 *   kind 1: clip_cov_loss_fn :238-261.  Means are masked_mean; candidates are the tokens with mask > 0 that
 *           the PPO clip leaves alone (pg_losses2 <= pg_losses1, bounds ratio_lo / ratio_hi as in
 *           axon_policy_loss) and whose covariance lies in (cov_lb, cov_ub);
 *           k = min(max(int(ratio * sum mask), 1), candidates) of them are selected uniformly at random
 *           (torch.randperm there; here the k largest of a hash of (token index, seed)).
 * keys [n_slots] (uint32) and state (axon_cov_select_state_bytes() bytes, 8-byte aligned) are outputs that
 * axon_cov_policy_loss reads; state starts with uint32 threshold, remaining, candidates, ties, then
 * int64 index_limit, float mean_a, mean_b, count, uint32 k.  Equal keys at the threshold go to the lowest
 * token indices (the reference leaves that order to the library).  workspace:
 * axon_cov_select_workspace_bytes(n_slots) bytes.  All arrays 16-byte aligned.  The histograms use integer
 * atomics only: the selection is reproducible. */
int64_t axon_cov_select_state_bytes(void);
int64_t axon_cov_select_workspace_bytes(int64_t n_slots);
int axon_cov_select(int kind, const float* logp, const float* old_logp, const float* adv,
                    const void* mask, int mask_kind, int64_t n_slots, double ratio, float cov_lb,
                    float cov_ub, float ratio_lo, float ratio_hi, uint32_t seed, uint32_t* keys,
                    void* state, void* workspace, void* stream);

/* The loss and gradient that go with axon_cov_select, aggregated as in axon_policy_loss (same row_scale /
 * uniform_scale / post_normalize / valid_count / acc / partials conventions):
 *   kind 0: kl_cov_loss_fn :303-345: -A*ratio, plus kl_coef * |clamped log ratio| on the selected tokens;
 *           acc[1] = sum mask*selected, acc[2] = sum mask*|clamped log ratio|
 *   kind 1: clip_cov_loss_fn :229-266: max(-A*ratio, -A*clamp(ratio)) with the selected tokens zeroed;
 *           acc[1] = sum mask*selected, acc[2] = sum mask*(-(clamped log ratio)) */
int axon_cov_policy_loss(int kind, const float* logp, const float* old_logp, const float* adv,
                         const void* mask, int mask_kind, const float* is_weights,
                         const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots,
                         int64_t uniform_len, const float* row_scale, float uniform_scale,
                         int post_normalize, const double* valid_count, float ratio_lo,
                         float ratio_hi, float kl_coef, const uint32_t* keys, const void* state,
                         float* grad, float* acc, float* partials, void* stream);

/* Per-token KL penalty against a reference policy, kl_penalty / kl_penalty_forward
 * (axon/utils/rl/kl.py:154-245): kl_type 1 "kl"/"k1", 2 "abs", 3 "mse"/"k2", 4 "low_var_kl"/"k3";
 * kl_plus != 0 for "k1+"/"k3+" (forward value of the type, gradient of k2, kl.py:184-190).
 * out[n] = the estimate, grad[n] = d out / d logp. */
int axon_kl_penalty(const float* logp, const float* ref_logp, int64_t n, int kl_type, int kl_plus,
                    float* out, float* grad, void* stream);

/* Entropy bonus and KL penalty of the actor loss, aggregated with agg_loss like the
 * policy-gradient term (CausalLM.forward_backward_fn, axon/models/fsdp_models.py:247-273), in one
 * pass: entropy (NULL: no entropy term), logp/ref_logp (kl_type 0: no KL term).
 * row_scale / uniform_scale / post_normalize / valid_count as in axon_policy_loss.
 * Outputs: agg_w[n_slots] = mask*scale (= d acc[0] / d entropy; may be NULL),
 * grad_kl[n_slots] = mask*scale * d kld / d logp (NULL when kl_type 0);
 * acc[8] (written): [0] aggregated entropy, [1] aggregated KL penalty, [2] sum entropy*mask,
 * [4] sum mask, [5] the factor the two gradient arrays still have to be multiplied by.
 * partials: workspace of axon_reduce_partials_bytes(n_slots). */
int axon_side_terms(const float* entropy, const float* logp, const float* ref_logp, const void* mask,
                    int mask_kind, const int32_t* cu_seqlens, int64_t n_rows, int64_t n_slots,
                    int64_t uniform_len, const float* row_scale, float uniform_scale,
                    int post_normalize, const double* valid_count, int kl_type, int kl_plus,
                    float* agg_w, float* grad_kl, float* acc, float* partials, void* stream);

/* GMPO, geo_mean_loss_fn (axon/trainer/algos/loss/loss.py:355-408): the sequence-level loss
 * -adv_r * exp(mean_t nak_min) * geo-mean(is_weights), averaged over rows that have tokens, with
 * its gradient w.r.t. logp.  clip_low / clip_high are the log-ratio clip ranges.
 * row_ws: 5 * n_rows floats, the first 4 * n_rows zero-filled by the caller.
 * acc[8] (written): [0] loss, [1] sum mask*(clipped & A>0), [2] sum mask*(old-logp),
 * [3] sum mask*(clipped & A<0), [4] sum mask.  partials: axon_reduce_partials_bytes(n_slots). */
int axon_gmpo_loss(const float* logp, const float* old_logp, const float* adv, const void* mask,
                   int mask_kind, const float* is_weights, const int32_t* cu_seqlens, int64_t n_rows,
                   int64_t n_slots, int64_t uniform_len, float clip_low, float clip_high, float* row_ws,
                   float* grad, float* acc, float* partials, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AXON_AMD_H */
