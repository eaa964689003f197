/*
 * vrl.h — C ABI of libvrl_hip.so: per-token scoring of LLM logits and the
 * SPEC-RL draft-verify step on one MI355X (gfx950).
 *
 * Conventions shared by every entry point
 *   - Every pointer named below is a DEVICE pointer into memory the caller
 *     owns (hipMalloc / torch allocator). The library allocates nothing,
 *     frees nothing and keeps no pointer after the call returns.
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).
 *     Kernels are enqueued on it and the call returns without synchronising.
 *   - Return value: VRL_OK, or a negative VRL_ERR_* found on the host before
 *     anything was enqueued (nothing has been launched in that case).
 *     Errors that only the device can see (a label outside [0, vocab)) are
 *     OR-ed into *err_flag (device int32, caller zeroes it, caller reads it
 *     after synchronising).
 *   - Nothing throws or aborts across this boundary.
 *   - First calls. The first call of an entry point on a device may touch the runtime beyond a launch: the
 *     matrix-core entry points (vrl_lmhead_score, vrl_lmhead_dlogits, vrl_gemm / vrl_gemm_nt) raise their kernels' LDS
 *     limit with hipFuncSetAttribute, once per device and kernel variant (element type, operand layouts, stored /
 *     accumulated / partial product, logits kept or not), and vrl_rowscore_split_static looks up its scratch array's
 *     address. Neither is allowed while a stream is being captured into a HIP graph: make each call once, with the
 *     options that will be captured, before the capture starts. Later calls only enqueue kernels.
 *   - Row space: logits are (n_rows, vocab), row r starts at element
 *     r * row_stride. Per-token arrays (labels, temperature, outputs, and
 *     for verify logp/mask/accept) are indexed by the same r.
 *   - Sequence space: sequence b owns rows [cu_seqlens[b], cu_seqlens[b+1])
 *     when cu_seqlens != NULL (packed layout, B+1 int64 entries), else rows
 *     [b*T, (b+1)*T) (padded (B, T) layout). `n_tokens` is the length of every
 *     per-token array: B*T for the padded layout (checked on the host). The
 *     packed offsets live on the device, so the kernels hold them to n_tokens:
 *     a span is cut to [0, n_tokens] before anything is indexed with it, and
 *     offsets that are not a partition of [0, n_tokens] set VRL_FLAG_SEQ_RANGE
 *     in *err_flag (the reference asserts the same, verl/workers/utils/padding.py:129-130).
 *     No access ever leaves the arrays, whatever cu_seqlens holds.
 */
#ifndef VRL_H_
#define VRL_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VRL_ABI_VERSION 4

/* status codes */
#define VRL_OK 0
#define VRL_ERR_NULL (-1)      /* a required pointer is NULL */
#define VRL_ERR_DTYPE (-2)     /* dtype is not one of VRL_F32 / VRL_BF16 / VRL_F16 */
#define VRL_ERR_SHAPE (-3)     /* negative count, vocab <= 0, stride < vocab, too many rows */
#define VRL_ERR_ALIGN (-4)     /* pointer not aligned to its element size */
#define VRL_ERR_HIP (-5)       /* the HIP runtime refused the launch; see vrl_last_hip_error */
#define VRL_ERR_ARG (-6)       /* inconsistent optional arguments */
#define VRL_ERR_SCRATCH (-7)   /* the request does not fit the library's static scratch (vrl_rowscore_split_static) */

/* logits element types */
#define VRL_F32 0
#define VRL_BF16 1
#define VRL_F16 2

/* bits of *err_flag */
#define VRL_FLAG_LABEL_OOB 1   /* some label was < 0 or >= vocab; that row's logprob is NaN */
#define VRL_FLAG_SLICE_RANGE 2 /* vrl_response_slice: a sequence had no prompt token or a bad response length */
#define VRL_FLAG_SEQ_RANGE 4   /* packed layout: cu_seqlens is not a partition of [0, n_tokens] (first entry != 0,
                                  last != n_tokens, decreasing, or out of range) */

/*
 * vrl_rowscore — one HBM pass over (n_rows, vocab) logits producing, per row,
 *   logprob[r]   = z[label[r]] - logsumexp(z)
 *   entropy[r]   = logsumexp(z) - sum(softmax(z) * z)
 *   sum_pi_sq[r] = sum(softmax(z)^2) = exp(logsumexp(2z) - 2 logsumexp(z))
 *   lse[r]       = logsumexp(z)            (what vrl_rowscore_backward needs)
 * with z = logits[r, :] / max(temperature[r], 1e-8) (z = logits[r, :] when
 * temperature == NULL), accumulated in fp32, written as fp32.
 *
 * Replaces, in the reference:
 *   verl/utils/torch_functional.py:73-107   logprobs_from_logits (dispatch)
 *   verl/utils/torch_functional.py:173-207  logprobs_from_logits_v2
 *   verl/utils/torch_functional.py:155-170  logprobs_from_logits_naive
 *   verl/utils/torch_functional.py:231-245  entropy_from_logits
 *   verl/utils/torch_functional.py:248-270  entropy_from_logits_with_chunking
 *   verl/utils/torch_functional.py:690-704  calculate_sum_pi_squared_from_logits
 *   verl/workers/engine/fsdp/transformer_impl.py:1357  division by per-token temperature
 *
 * Each output pointer may be NULL to skip that output (labels may be NULL when
 * out_logprob is); at least one must be given.
 * Rows containing -inf logits give NaN entropy (0 * -inf), as torch does.
 */
int vrl_rowscore(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                 const int64_t* labels, const float* temperature, float* out_logprob,
                 float* out_entropy, float* out_sum_pi_sq, float* out_lse, int32_t* err_flag,
                 void* stream);

/*
 * vrl_label_logprob — log-probs of the labels from a logsumexp that an earlier pass over the same rows left behind:
 *   logprob[r] = z[label[r]] - lse[r],   z as in vrl_rowscore
 * One element load per row instead of a pass over the row: what a caller runs when it asked vrl_rowscore for the
 * entropy (and out_lse) first and needs the label log-probs of the same logits afterwards, which is the order of the
 * reference's engine (verl/workers/engine/fsdp/transformer_impl.py:1364-1376 entropy, :1395-1399 log-probs). The
 * result is within one rounding of lse (fp32) of what vrl_rowscore writes to out_logprob. A label outside [0, vocab)
 * gives NaN and VRL_FLAG_LABEL_OOB. Replaces the gather of verl/utils/torch_functional.py:194-198.
 */
int vrl_label_logprob(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                      const int64_t* labels, const float* temperature, const float* lse, float* out_logprob,
                      int32_t* err_flag, void* stream);

/*
 * vrl_rowscore_split — the same results for FEW rows: n_splits workgroups share
 * each row and a second small kernel merges their partial results, so that a
 * batch of tens or hundreds of rows still occupies the whole chip.
 * `partials` is caller-owned scratch of n_rows * n_splits * 4 floats; its
 * contents before and after the call are meaningless. n_splits in [1, 64];
 * n_splits == 1 is vrl_rowscore. vrl_rowscore_split_plan returns the n_splits
 * this library would pick for a shape (1 = do not split), so a caller can size
 * the scratch before the call. Same reference counterparts as vrl_rowscore.
 */
int vrl_rowscore_split(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                       const int64_t* labels, const float* temperature, float* out_logprob,
                       float* out_entropy, float* out_sum_pi_sq, float* out_lse, int32_t* err_flag,
                       int n_splits, float* partials, void* stream);
int vrl_rowscore_split_plan(int dtype, int64_t n_rows, int64_t vocab);

/*
 * vrl_rowscore_split_static — vrl_rowscore_split for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference.
 * Same arguments and results (bit for bit) as vrl_rowscore_split minus `partials`: the partial results live in
 * a static device array inside the library of VRL_STATIC_PARTIALS_MAX (row, slice) entries of 16 bytes
 * (128 KiB on every GPU the library runs on, held until the process ends). n_rows * n_splits beyond that
 * returns VRL_ERR_SCRATCH and launches nothing (n_splits == 1 needs no scratch and takes any n_rows).
 * The call allocates and frees nothing. Every call on one GPU shares that GPU's array: calls that overlap in
 * time on one GPU (two streams, two threads) race and must be serialised by the caller; calls on different
 * GPUs are independent. The first call on a device looks the array's address up (hipGetSymbolAddress), so
 * make one call outside any graph capture first.
 */
#define VRL_STATIC_PARTIALS_MAX 8192
int vrl_rowscore_split_static(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                              const int64_t* labels, const float* temperature, float* out_logprob,
                              float* out_entropy, float* out_sum_pi_sq, float* out_lse, int32_t* err_flag,
                              int n_splits, void* stream);

/*
 * vrl_rowscore_backward — gradient of the row op with respect to the logits,
 * one read of the logits and one write of the gradient (same dtype as the logits):
 *   dlogits[r, v] = ( g_logprob[r] * (1[v == label[r]] - p)  -  g_entropy[r] * p * (log p + entropy[r]) ) / T[r]
 * with p = exp(z_v - lse[r]), z = logits[r, :] / max(temperature[r], 1e-8). `lse` and
 * `entropy` are the forward outputs. g_logprob or g_entropy may be NULL (that
 * term is then absent; labels / entropy may be NULL with it). dlogits may be
 * the logits buffer itself (in place). Elements whose p underflows to 0 get 0.
 *
 * Replaces what torch autograd builds for the compositions at
 *   verl/workers/engine/fsdp/transformer_impl.py:1357-1399 under update_actor
 *   (verl/workers/engine_workers.py:707-714, loss.backward() at fsdp/transformer_impl.py:739-743);
 * the closed form is the reference's verl/utils/experimental/torch_functional.py:66-79.
 */
int vrl_rowscore_backward(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                          const int64_t* labels, const float* temperature, const float* lse,
                          const float* entropy, const float* g_logprob, const float* g_entropy,
                          void* dlogits, int64_t d_row_stride, void* stream);

/*
 * vrl_score_responses — ONE launch from packed logits (n_rows, vocab) to the padded (B, T_out) response blocks:
 *   label[r]           = labels[r], or input_ids[(r + 1) mod n_rows] when input_ids is given instead
 *                        (the roll of verl/workers/engine/fsdp/transformer_impl.py:1177; exactly one of the two,
 *                        or neither when only the entropy is asked for)
 *   logprob / entropy  as vrl_rowscore
 *   resp_logprob[b, j] = logprob[cu_seqlens[b+1] - response_lens[b] - 1 + j]  for j < response_lens[b], else 0
 *   resp_entropy[b, j] likewise            (the left shift by one of verl/workers/utils/padding.py:135-138)
 * resp_logprob / resp_entropy: at least one; resp_lse (optional) receives the logsumexp in the same layout, which is what
 * vrl_score_responses_backward needs. out_logprob / out_entropy (n_rows, per token) are optional extras of the
 * block of the same kind; when neither is given, rows outside every response window are not read at all (a prompt
 * token's logits cost no memory traffic).
 * Device-side checks, reported through *err_flag: a label outside [0, vocab) (VRL_FLAG_LABEL_OOB, that entry NaN);
 * a sequence without a prompt token or with response_lens[b] outside [0, T_out] (VRL_FLAG_SLICE_RANGE, its row all
 * zero); cu_seqlens not a partition of [0, n_rows] (VRL_FLAG_SEQ_RANGE, the offending sequences' rows all zero).
 * No content of cu_seqlens or response_lens can make the kernel touch memory outside the arrays.
 *
 * Replaces, as one kernel, the sequence
 *   verl/workers/engine/fsdp/transformer_impl.py:1177 (labels = roll(input_ids, -1)), :1357 (temperature),
 *   :1364-1399 (entropy, log-probs), :1401-1418 + verl/workers/utils/padding.py:97-141 (no_padding_2_padding).
 */
int vrl_score_responses(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                        const int64_t* labels, const int64_t* input_ids, const float* temperature,
                        const int64_t* cu_seqlens, const int64_t* response_lens, int64_t B, int64_t T_out,
                        float* out_logprob, float* out_entropy, float* resp_logprob, float* resp_entropy,
                        float* resp_lse, int32_t* err_flag, void* stream);

/*
 * vrl_score_responses_backward — gradient of vrl_score_responses with respect to the logits, from the gradients of the
 * two (B, T_out) blocks: row r inside the response window of sequence b (column j) gets
 *   dlogits[r, :] = vrl_rowscore_backward's row for g_logprob = g_resp_logprob[b, j], g_entropy = g_resp_entropy[b, j],
 *                   lse = resp_lse[b, j], entropy = resp_entropy[b, j]
 * (resp_lse is the optional logsumexp block of the forward call), every other row zeros, written without reading that
 * row's logits. dlogits has the logits' type and may be the logits buffer itself. g_resp_logprob or g_resp_entropy
 * may be NULL. Labels as in the forward call (labels, or input_ids rolled by one). Offsets that fail the forward call's
 * validation give zero rows here; they were reported there.
 *
 * Replaces what autograd builds for verl/workers/engine/fsdp/transformer_impl.py:1177,1357-1418 +
 * verl/workers/utils/padding.py:97-141 under update_actor.
 */
int vrl_score_responses_backward(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                 const int64_t* labels, const int64_t* input_ids, const float* temperature,
                                 const int64_t* cu_seqlens, const int64_t* response_lens, int64_t B, int64_t T_out,
                                 const float* resp_lse, const float* resp_entropy, const float* g_resp_logprob,
                                 const float* g_resp_entropy, void* dlogits, int64_t d_row_stride, void* stream);

/*
 * vrl_response_slice — packed per-token values (total_nnz, *) -> padded (B, T_out, *)
 * response block: out[b, j] = values[cu_seqlens[b+1] - response_lens[b] - 1 + j]
 * for j < response_lens[b], else zeros (the model output at a position scores the
 * NEXT token, hence the shift by one). A value is a row of row_bytes bytes: the
 * element size times the product of the trailing dimensions (4 for an fp32 vector,
 * 2 * K for (total_nnz, K) bf16 top-k log-probs, ...), copied bit for bit, whatever
 * the element type; the trailing dimensions are not padded
 * (verl/workers/utils/padding.py:100-101, :133-138: skip_padding = (0, 0) * (values.ndim - 1)).
 * `values` has n_tokens rows, out B * T_out rows; neither needs more alignment than its element type. Sets
 * VRL_FLAG_SLICE_RANGE and writes a zero row block when a sequence has no prompt token,
 * or response_lens[b] is outside [0, T_out]; VRL_FLAG_SEQ_RANGE and a zero row block when
 * the sequence's offsets do not fit n_tokens (see "Sequence space" above).
 * row_bytes is at most 2^30; T_out * row_bytes at most 2^31 or so (VRL_ERR_SHAPE beyond).
 *
 * Replaces verl/workers/utils/padding.py:97-141 (no_padding_2_padding); fixture:
 * tests/models/test_fsdp_no_padding_on_gpu.py:180-201.
 */
int vrl_response_slice(const void* values, int64_t row_bytes, const int64_t* cu_seqlens, const int64_t* response_lens,
                       int64_t B, int64_t n_tokens, int64_t T_out, void* out, int32_t* err_flag, void* stream);

/*
 * vrl_expand_per_sequence — one fp32 value per sequence -> one per token of the packed batch:
 *   out[t] = values[b]  for  cu_seqlens[b] <= t < cu_seqlens[b+1]
 * (empty sequences contribute nothing). This is how the engine turns the per-sample temperature into the per-token
 * one that the scoring entry points take. `values` has B entries, `out` n_tokens. Offsets that are not a partition of
 * [0, n_tokens] set VRL_FLAG_SEQ_RANGE; a token that no sequence holds gets 0. B = 0 with n_tokens > 0 is
 * VRL_ERR_SHAPE.
 *
 * Replaces verl/utils/torch_functional.py:989-1011 (expand_as_nested: repeat_interleave by the sequence lengths) as
 * called at verl/workers/engine/fsdp/transformer_impl.py:1158-1162.
 */
int vrl_expand_per_sequence(const float* values, const int64_t* cu_seqlens, int64_t B, int64_t n_tokens, float* out,
                            int32_t* err_flag, void* stream);

/*
 * vrl_response_pack — packed per-token values (total_nnz, *) -> packed response values (sum of response_lens, *):
 *   out[out_offsets[b] + j] = values[cu_seqlens[b+1] - response_lens[b] - 1 + j],  j < response_lens[b]
 * with rows of row_bytes bytes as in vrl_response_slice.
 * out_offsets is the caller's exclusive prefix sum of response_lens (B+1 entries, last = out_total rows).
 * A sequence without a prompt token, a negative length, or a window that is not exactly
 * [out_offsets[b], out_offsets[b+1]) inside the output (the last one ending at out_total) sets VRL_FLAG_SLICE_RANGE
 * and writes nothing for it;
 * offsets that do not fit the n_tokens rows of `values` set VRL_FLAG_SEQ_RANGE and write nothing for it.
 *
 * Replaces verl/workers/utils/padding.py:194-210 (response_from_nested).
 */
int vrl_response_pack(const void* values, int64_t row_bytes, const int64_t* cu_seqlens, const int64_t* response_lens,
                      const int64_t* out_offsets, int64_t B, int64_t n_tokens, int64_t out_total, void* out,
                      int32_t* err_flag, void* stream);

/*
 * vrl_transpose — out-of-place transposition of a 2-D array of 2-byte (bf16, fp16) or
 * 4-byte (fp32) elements, bit for bit:
 *   dst[c * dst_stride + r] = src[r * src_stride + c],   r < rows, c < cols
 * (strides in elements; src_stride >= cols, dst_stride >= rows; the arrays must not overlap).
 *
 * Serves the backward of the LM head + scoring step: the reference forms
 *   dhidden = dlogits @ vocab_weights,  dvocab_weights = dlogits.t() @ hidden_states
 *   (verl/utils/experimental/torch_functional.py:80-81)
 * on the operands as stored; the library GEMM on this part runs those products 25-35 % faster when
 * both operands are contiguous along the contraction axis, which one transposition of the weight
 * (per backward) and of the hidden-state chunk provides.
 */
int vrl_transpose(const void* src, int elem_size, int64_t rows, int64_t cols, int64_t src_stride,
                  void* dst, int64_t dst_stride, void* stream);

/*
 * vrl_lmhead_score — LM head and scoring in one pass on the matrix cores, without logits in memory:
 *   z[t, v] = (sum_k hidden[t, k] * weight[v, k]) / max(temperature[t], 1e-8)
 *   logprob[t] = z[t, label[t]] - logsumexp(z[t, :]),  entropy[t] = logsumexp - sum(softmax * z),  lse[t] = logsumexp
 * hidden (n_tokens, hidden_size) and weight (vocab, hidden_size) are bf16 or fp16 (dtype as for vrl_rowscore),
 * row-major with row pitches h_stride / w_stride in elements; products are accumulated in fp32 (the logits are
 * NOT rounded to the operand type on the way, unlike a GEMM that writes them out). Forward only.
 * `partials` is caller-owned scratch of vrl_lmhead_partials(n_tokens, vocab) floats (12 per token and 768 vocabulary
 * entries); vrl_lmhead_plan gives n_splits, which only decides how the work is dealt to workgroups: a token's softmax
 * state is handed over at fixed places of the vocabulary and merged in a fixed order, so its results are the same bits
 * for any n_splits and any number of tokens in the call.
 * Requirements checked on the host: n_tokens >= 256, vocab >= 256, hidden_size a multiple of 64, pitches multiples
 * of 8 elements and at most 2^28, n_tokens and vocab at most 2^30, 16-byte aligned operands, 1 <= n_splits <= 64. out_logprob (with labels
 * and err_flag), out_entropy, out_lse: any may be NULL, not all.
 * logits_out (optional): the logits themselves, sum_k hidden[t, k] * weight[v, k] before the temperature, rounded once to the
 * operands' type and written to logits_out[t * logits_stride + v] from the registers that hold them (vocab and logits_stride
 * multiples of 8, 16-byte aligned): for a backward pass that may spend n_tokens * vocab elements of memory instead of
 * forming the logits again, which then runs vrl_rowscore_backward over them in place (the reference's torch path keeps
 * them the same way, verl/utils/experimental/torch_functional.py:33-35). The scores are folded from the fp32 values either way.
 * Only the first logits_rows tokens' logits are written (1 <= logits_rows <= n_tokens, VRL_ERR_SHAPE otherwise; ignored
 * without logits_out): a caller with a memory budget keeps what fits and forms the rest again in its backward pass.
 *
 * fp32 operands are refused (VRL_ERR_DTYPE) on purpose: the part's fp32 matrix rate (157 TFLOP/s) is what the library GEMM
 * already delivers, so an fp32 LM head is served by the library GEMM followed by vrl_rowscore (the Python side does that),
 * where the reference's Triton loop takes any element type (verl/utils/kernel/kernels.py:183-188).
 *
 * Replaces the reference's fused linear + cross-entropy forward:
 *   verl/utils/kernel/linear_cross_entropy.py:38-85 (LinearCrossEntropy.forward)
 *   verl/utils/kernel/kernels.py:183-451 (efficient_entropy_kernel_general_mainloop + epilogue, Triton)
 */
int vrl_lmhead_score(const void* hidden, const void* weight, int dtype, int64_t n_tokens, int64_t vocab,
                     int64_t hidden_size, int64_t h_stride, int64_t w_stride, const int64_t* labels,
                     const float* temperature, int n_splits, float* partials, float* out_logprob,
                     float* out_entropy, float* out_lse, int32_t* err_flag, void* logits_out, int64_t logits_stride,
                     int64_t logits_rows, void* stream);
/*
 * vrl_lmhead_dlogits — backward counterpart of vrl_lmhead_score: the logits are formed again on the matrix cores,
 * tile by tile, and turned in registers into the gradient with respect to the logits,
 *   dlogits[t, v] = ( g_logprob[t] * (1[v == label[t]] - p)  -  g_entropy[t] * p * (log p + entropy[t]) ) / T[t],
 *   p = exp(z[t, v] - lse[t]),  z as in vrl_lmhead_score
 * (the arithmetic of vrl_rowscore_backward on fp32 logits that were never rounded to the operand type), which is
 * written in the operands' type to dlogits[t * d_stride + v], t < n_tokens, v < vocab. The caller forms
 *   d hidden = dlogits @ weight,   d weight = dlogits^T @ hidden
 * with its GEMM of choice, as the reference does (torch.matmul at verl/utils/kernel/kernels.py:1710-1720).
 * lse and entropy are vrl_lmhead_score's outputs. g_logprob or g_entropy may be NULL (that term is then absent;
 * labels / entropy may be NULL with it). Same shape rules as vrl_lmhead_score, plus vocab and d_stride multiples
 * of 8 and a 16-byte aligned dlogits. n_splits as from vrl_lmhead_plan. No scratch.
 *
 * Replaces the reference's default backward kernel of the fused linear + cross-entropy op:
 *   verl/utils/kernel/kernels.py:1229-1387 (efficient_entropy_backward_kernel_general_d_logits_split_N, Triton)
 *   and its host loop :1663-1721 (BackwardEnum._Split_Dlogits_N).
 */
int vrl_lmhead_dlogits(const void* hidden, const void* weight, int dtype, int64_t n_tokens, int64_t vocab,
                       int64_t hidden_size, int64_t h_stride, int64_t w_stride, const int64_t* labels,
                       const float* temperature, const float* lse, const float* entropy, const float* g_logprob,
                       const float* g_entropy, int n_splits, void* dlogits, int64_t d_stride, void* stream);

/*
 * vrl_gemm — out[y][x] (+)= sum_k X[x][k] * Y[y][k] on the matrix cores, with the main loop of the LM-head kernels: the
 * two products that follow vrl_lmhead_dlogits in the backward, read from the tensors as they lie,
 *   d hidden (tokens, hidden) = G . W      : x = W (vocab, hidden), contraction-major; y = G (tokens, vocab), row-major
 *   d W      (vocab, hidden) += G^T . H    : x = H (tokens, hidden) and y = G (tokens, vocab), both contraction-major,
 *                                            accumulate = 1 from the second chunk of tokens on.
 * A row-major operand is (N, K), contiguous along the contraction, with row stride >= K; a contraction-major one
 * (x_contraction_major / y_contraction_major != 0) is (K, N), contiguous along its N rows, with row stride >= N and N a
 * multiple of 8. Strides are in elements and multiples of 8, bases 16-byte aligned. out is (NY, NX) in the operands' type
 * (VRL_BF16 or VRL_F16) with row stride out_stride (a multiple of 4, 8-byte aligned base); fp32 accumulation, one
 * rounding; the result does not depend on the operands' layouts. NX, NY >= 256, NX a multiple of 4, K a multiple of 64
 * and >= 128; strides at most 2^28 elements, NX, NY and K at most 2^30. accumulate != 0 adds the product to what out holds.
 * k_parts (1..16, normally what vrl_gemm_nt_plan returns) cuts the contraction into ranges that are summed in a fixed
 * order through `workspace` (k_parts * NX * NY floats, 16-byte aligned; may be NULL when k_parts == 1): that is how a
 * product with few output tiles still fills the CUs. vrl_gemm_nt_plan returns the number of ranges it would use for a
 * shape (or a negative status) and stores the workspace it needs. vrl_gemm_nt is vrl_gemm for two row-major operands.
 *
 * Replaces the two torch.matmul calls of the reference's backward (verl/utils/kernel/kernels.py:1710-1720).
 */
int vrl_gemm_nt_plan(int dtype, int64_t NX, int64_t NY, int64_t K, int64_t* workspace_floats);
int vrl_gemm(const void* x, const void* y, int dtype, int64_t NX, int64_t NY, int64_t K, int64_t x_stride,
             int64_t y_stride, int x_contraction_major, int y_contraction_major, void* out, int64_t out_stride,
             int accumulate, int k_parts, float* workspace, void* stream);
int vrl_gemm_nt(const void* x, const void* y, int dtype, int64_t NX, int64_t NY, int64_t K, int64_t x_stride,
                int64_t y_stride, void* out, int64_t out_stride, int accumulate, int k_parts, float* workspace,
                void* stream);
/* Vocabulary splits per 256-token block for this shape: the number (at most 64) for which the workgroups, one per CU
 * at a time, finish soonest: rounds of workgroups times the vocabulary tiles of the longest share. Results do not
 * depend on it. vrl_lmhead_partials: floats of scratch that vrl_lmhead_score needs for this shape. */
int vrl_lmhead_plan(int64_t n_tokens, int64_t vocab);
int64_t vrl_lmhead_partials(int64_t n_tokens, int64_t vocab);

/*
 * vrl_rollout_corr — rollout correction on padded (B, T) log-probs in one launch:
 *   lr = clamp(old - rollout, +-20);  k1 = -lr, k2 = lr^2/2, k3 = exp(lr) - 1 - lr
 *   keep[b,t]    = every enabled criterion passes (token_k1/k2/k3 per token; seq_sum / seq_mean /
 *                  seq_max of k1/k2/k3 per sequence; k1 criteria are two-sided [lo, hi], the others <= hi)
 *   weights[b,t] = mask * exp(lr)  (is_mode 1)  or  mask * exp(clamp(sum_t lr, +-20))  (is_mode 2),
 *                  then min(w, is_upper) (icepop 0) or zeroed outside [is_lower, is_upper] (icepop 1)
 *   stats[b, :]  = vrl_rollout_corr_num_stats() per-sequence partial sums / extrema (layout: enum CorrStat in
 *                  verl_amd/csrc/rollout_corr_kernels.h), enough to derive every metric of the step
 *   seq_keep_bits[b] = bit i set when the sequence passes enabled sequence-level criterion i
 * rs_bits: bit i enables criterion i in the order token_k1, token_k2, token_k3, seq_sum_k1..k3,
 * seq_mean_k1..k3, seq_max_k2, seq_max_k3. rs_lo_host / rs_hi_host are HOST arrays of 11 floats holding the
 * bounds as they are compared (natural log of the ratio bounds for k1 criteria). weights and keep may be NULL.
 *
 * Replaces the tensor work of verl/trainer/ppo/rollout_corr_helper.py:
 *   compute_rollout_rejection_mask :197-413, compute_rollout_correction_weights :522-657,
 *   compute_offpolicy_metrics :904-1010 (and the per-element parts of compute_rs_metrics :416-519 and
 *   compute_is_metrics :660-783); the scalar metrics are finished on the host from `stats`.
 */
int vrl_rollout_corr(const float* old_log_prob, const float* rollout_log_prob, const uint8_t* mask, int64_t B,
                     int64_t T, int is_mode, int icepop, float is_upper, float is_lower, float is_lower_metric,
                     uint32_t rs_bits, const float* rs_lo_host, const float* rs_hi_host, float* weights,
                     uint8_t* keep, float* stats, int32_t* seq_keep_bits, void* stream);
int vrl_rollout_corr_num_stats(void);

/*
 * vrl_spec_verify — SPEC-RL draft verification over B sequences.
 * For token i of sequence b:
 *   d = logp_new[i] - logp_old[i];  tau = log_u[i] + thresh_offset      (fp32, no contraction)
 *   valid = mask ? mask[i] != 0 : 1
 *   accept[i] = valid && d >= tau            (NaN compares false => reject)
 *   first_reject[b] = smallest in-sequence position with valid && !(d >= tau);
 *                     when there is none, one past the last valid position
 *                     (= number of valid tokens for a right-padded mask)
 *   prefix_len[b]   = number of valid tokens at positions < first_reject[b]
 *   near_count[b]   = number of valid tokens with |d - tau| < near_eps
 * Optional truncated draft (all three or none): for positions >= first_reject
 *   out_ids = pad_id, out_mask = 0; below it they copy draft_ids / mask.
 * err_flag is required for the packed layout (VRL_FLAG_SEQ_RANGE) and may be NULL for the padded one.
 *
 * Two forms, chosen by `workspace`:
 *   workspace == NULL (workspace_bytes 0): one launch, one workgroup per sequence. Right for batches of sequences of
 *     similar, moderate length. Tokens that no in-range span covers are not written (packed layout, bad offsets).
 *   workspace != NULL: two launches that walk the token arrays in tiles of 1024 tokens whatever sequence a token
 *     belongs to, so that no CU is left with a long sequence's bytes (512 packed sequences of 32 ... 16384 tokens:
 *     the per-sequence form takes as long as its longest sequences' CUs). What a sequence needs from its other tiles
 *     travels through `workspace` as four bits per token: caller-owned device scratch of at least
 *     vrl_spec_verify_workspace(n_tokens) bytes (0.5 bytes per token), 8-byte aligned, contents meaningless before
 *     and after. accept is written for every token of the arrays. Same integers as the other form.
 * vrl_spec_verify_plan returns 1 when the library would take the second form for a shape (packed != 0: cu_seqlens
 * given), so a caller can size the scratch before the call; passing a workspace is what selects it.
 *
 * No function in the reference computes this (its recipe/ submodule is not
 * vendored: .gitmodules:1-3). Layout, mask and sign conventions follow
 *   verl/trainer/ppo/rollout_corr_helper.py:197-233,262-268,849
 *   verl/trainer/ppo/ray_trainer.py:120-135 (response_mask = attention_mask[:, -T:])
 * which is where a caller would slot it in (ray_trainer.py:1647-1660).
 */
int vrl_spec_verify(const float* logp_new, const float* logp_old, const float* log_u,
                    const uint8_t* mask, const int64_t* cu_seqlens, int64_t B, int64_t T, int64_t n_tokens,
                    float thresh_offset, float near_eps, uint8_t* accept, int32_t* first_reject,
                    int32_t* prefix_len, int32_t* near_count, const int64_t* draft_ids,
                    int64_t pad_id, int64_t* out_ids, uint8_t* out_mask, int32_t* err_flag, void* workspace,
                    int64_t workspace_bytes, void* stream);
int64_t vrl_spec_verify_workspace(int64_t n_tokens);
int vrl_spec_verify_plan(int packed, int64_t B, int64_t T, int64_t n_tokens);

/*
 * vrl_truncate_draft — apply an already known first_reject[b] to a draft:
 * positions >= first_reject[b] get pad_id / mask 0, the rest are copied.
 * Same provenance as vrl_spec_verify (no reference counterpart); the nearest
 * reference step is the mask rewrite at verl/trainer/ppo/rollout_corr_helper.py:1061.
 */
int vrl_truncate_draft(const int64_t* draft_ids, const uint8_t* mask, const int64_t* cu_seqlens,
                       int64_t B, int64_t T, int64_t n_tokens, const int32_t* first_reject, int64_t pad_id,
                       int64_t* out_ids, uint8_t* out_mask, int32_t* err_flag, void* stream);

/*
 * vrl_fused_score_verify — scoring and verification of the same batch in one
 * call: the results of vrl_rowscore, and of vrl_spec_verify fed with the
 * log-probs just computed (logp_new = out_logprob, which is therefore required).
 * Row space and sequence space are as above with n_tokens = n_rows: the host
 * checks n_rows == B*T (padded); the verify kernel holds the packed offsets to
 * n_rows and reports VRL_FLAG_SEQ_RANGE through the same err_flag.
 *
 * Two launches on `stream`: the row kernel, then the verify kernel in its one-workgroup-per-sequence form (a caller
 * with widely differing sequence lengths calls vrl_rowscore and vrl_spec_verify with a workspace instead). (Doing the
 * verification inside the row kernel, by the last workgroup of each sequence,
 * was measured and is slower on MI355X: the agent-scope release each workgroup
 * needs costs more than the second launch.)
 *
 * Replaces the composition at
 *   verl/workers/engine/fsdp/transformer_impl.py:1353-1399 (divide, entropy, log-probs)
 * plus the verify step described under vrl_spec_verify.
 */
int vrl_fused_score_verify(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                           int64_t row_stride, const int64_t* labels, const float* temperature,
                           float* out_logprob, float* out_entropy, float* out_sum_pi_sq, float* out_lse,
                           int32_t* err_flag, const float* logp_old, const float* log_u, const uint8_t* mask,
                           const int64_t* cu_seqlens, int64_t B, int64_t T, float thresh_offset,
                           float near_eps, uint8_t* accept, int32_t* first_reject,
                           int32_t* prefix_len, int32_t* near_count, const int64_t* draft_ids,
                           int64_t pad_id, int64_t* out_ids, uint8_t* out_mask, void* stream);

/* Text for a VRL_* status code; never NULL. */
const char* vrl_strerror(int status);

/* hipGetErrorString of the last launch this thread saw refused ("" if none). */
const char* vrl_last_hip_error(void);

/* VRL_ABI_VERSION the library was built with. */
int vrl_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* VRL_H_ */
