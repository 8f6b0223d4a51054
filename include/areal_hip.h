/* C ABI of libareal_hip.so: MI355X (gfx950) kernels for AReaL's per-token RL training hot path.
 *
 * Conventions
 *   - every pointer is a device pointer unless stated otherwise; the library never allocates,
 *     never synchronises and only touches the stream it is given;
 *   - scratch memory is passed in by the caller (`workspace`, sized by the matching
 *     *_workspace_bytes function);
 *   - return value 0 = success, negative = error (see areal_status);
 *   - bf16 tensors are passed as `const void*` (raw bfloat16 bit patterns), masks as uint8_t
 *     (0/1, the memory layout of torch.bool).
 *
 * The reference (areal-project/AReaL) is pure Python and has no FFI for this path; each entry
 * point cites the Python function it replaces (paths relative to the reference root).
 */
#ifndef AREAL_HIP_H
#define AREAL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* areal_stream_t; /* a hipStream_t */

/* Version of this interface. It moves whenever an entry point's argument list or the size of a
 * caller-allocated buffer changes; a caller built against another number must not call in.
 * areal_abi_version() returns the number the loaded library was built with.
 *   3: areal_lmhead_fwd / areal_lmhead_bwd_saved take probs_bytes and check it against
 *      areal_lmhead_probs_bytes() (the buffer's rows are padded to 128, and
 *      areal_lmhead_bwd_saved takes probs_status); areal_sapo_loss takes entropy, extra0,
 *      extra1 and stats. */
#define AREAL_HIP_ABI_VERSION 3
int areal_abi_version(void);

enum areal_status {
  AREAL_OK = 0,
  AREAL_ERR_BAD_ARG = -1,
  AREAL_ERR_ALIGNMENT = -2,
  AREAL_ERR_WORKSPACE = -3,
  AREAL_ERR_LAUNCH = -4,
  AREAL_ERR_UNSUPPORTED = -5
};

/* ---------------------------------------------------------------------------------------
 * Fused lm_head -> log-softmax -> label log-prob + entropy
 * replaces _ChunkedVocabParallelLMHead.forward / .backward
 * (areal/models/mcore/vocab_parallel_head.py:564-735, :737-938) and the
 * torch.mm(..., out_dtype=float32) contraction of _linear_chunk_fp32 (:538-557).
 * ------------------------------------------------------------------------------------- */

size_t areal_lmhead_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V);

/* Bytes of the bf16 buffer of saved softmax exponentials (`probs` below):
 * round_up(T, 128) rows of round_up(V, 64) columns. */
size_t areal_lmhead_probs_bytes(int64_t T, int64_t V);

/* hidden [T,H] bf16, weight [V,H] bf16 (H % 8 == 0, 16-byte aligned), bias [V] fp32 or NULL,
 * labels [T] int64. Outputs fp32 [T]; row_max and sum_exp are the state saved for backward
 * (vocab_parallel_head.py:704-713). logits = (hidden . weight^T + bias) * logit_scale.
 *
 * probs / probs_ref / probs_status (all NULL, or all set) additionally keep the softmax
 * exponentials for areal_lmhead_bwd_saved, the counterpart of autograd saving the logits in the
 * reference's logits-in path (_gather_logprobs_entropy,
 * areal/utils/functional/vocab_parallel.py:24-30): probs is bf16
 * [round_up(T,128)][round_up(V,64)] (probs_bytes = its size in bytes, at least
 * areal_lmhead_probs_bytes(T, V), else AREAL_ERR_WORKSPACE) holding
 * 2^(x / T * log2(e) - probs_ref[t]); probs_ref is
 * fp32 [T], a per-row reference estimated from a few logits of the row (its label's among
 * them) before the sweep; *probs_status (one int32 on the device) is written 0 when every
 * row's exponentials are in range, 1 when some row's maximum lies more than 100 binades (69 nats
 * at temperature 1) above its estimate: probs must then not be used and the backward recomputes
 * (areal_lmhead_bwd). The per-token outputs are right in both cases: when the status comes out
 * 1 the sweep is repeated without saving inside this call (launches queued behind the first
 * sweep that return at once otherwise), no host synchronisation involved. */
int areal_lmhead_fwd(const void* hidden, const void* weight, const float* bias,
                     const int64_t* labels, int64_t T, int64_t H, int64_t V,
                     float inv_temperature, float logit_scale, float* logprobs, float* entropy,
                     float* vocab_min, float* vocab_max, float* vocab_mean, float* vocab_norm,
                     float* row_max, float* sum_exp, void* probs, size_t probs_bytes,
                     float* probs_ref, int* probs_status, void* workspace, size_t workspace_bytes,
                     areal_stream_t stream);

size_t areal_lmhead_bwd_workspace_bytes(int64_t T, int64_t H, int64_t V, int64_t token_chunk);

/* grad_logprobs [T] fp32. Writes dhidden [T,H] bf16 (NULL to skip) and dweight [V,H] (NULL to
 * skip): fp32 overwritten (accumulate 0) or added to (accumulate 1, Megatron's main_grad,
 * vocab_parallel_head.py:873-879), or bf16 written by the contraction itself (accumulate 2;
 * only with token_chunk >= T, else AREAL_ERR_UNSUPPORTED: several chunks need the fp32 sum);
 * dbias [V] fp32 (NULL to skip; added to when accumulate is 1) = column sums of dlogits
 * (vocab_parallel_head.py:862-863). dlogits are rounded to bf16 before the gradient
 * contractions, as in vocab_parallel_head.py:830-839. */
int areal_lmhead_bwd(const void* hidden, const void* weight, const float* bias,
                     const int64_t* labels, const float* row_max, const float* sum_exp,
                     const float* grad_logprobs, int64_t T, int64_t H, int64_t V,
                     float inv_temperature, float logit_scale, void* dhidden, void* dweight,
                     float* dbias, int accumulate, int64_t token_chunk, void* workspace,
                     size_t workspace_bytes, areal_stream_t stream);

size_t areal_lmhead_bwd_saved_workspace_bytes(int64_t T, int64_t H, int64_t V);

/* Backward from the exponentials the forward kept (probs, probs_ref, *probs_status read back as
 * 0): the logits are not recomputed (vocab_parallel_head.py:806-829 recomputes them chunk by
 * chunk to save memory; an MI355X has the HBM to keep them) and no pass rewrites the [T, V]
 * buffer: dlogits[t][:] = f[t] * probs[t][:] with a per-row factor that dHidden applies to its
 * output rows and dWeight to the hidden states. Only the label's entry of each row of probs is
 * rewritten (and rows [T, round_up(T, 128)) are cleared), so probs can be used once; probs_bytes
 * as in areal_lmhead_fwd. logprobs (NULL allowed) are the forward's label
 * log-probabilities: with them the label's dlogit is -expm1(logprob) in fp32. dweight [V,H]:
 * dweight_mode 0 = fp32 store, 1 = fp32 accumulate, 2 = bf16 store; dbias [V] fp32 or NULL
 * (added to in mode 1). Other arguments as areal_lmhead_bwd; the bias itself does not enter (it
 * is part of the saved exponentials). probs_status (NULL allowed): the device int the forward
 * set; when it reads non-zero at execution time every kernel of this call returns at once and
 * no output is touched, so the call can be queued before the host has seen the status (the
 * caller then checks it and runs areal_lmhead_bwd instead if it was set). */
int areal_lmhead_bwd_saved(const void* hidden, const void* weight, const int64_t* labels,
                           const float* row_max, const float* sum_exp, const float* logprobs,
                           const float* grad_logprobs, int64_t T, int64_t H, int64_t V,
                           float inv_temperature, float logit_scale, void* probs, size_t probs_bytes,
                           const float* probs_ref, const int* probs_status, void* dhidden, void* dweight,
                           int dweight_mode, float* dbias, void* workspace,
                           size_t workspace_bytes, areal_stream_t stream);

/* out[j*ldo + i] = sum_k A[i*lda + k] * B[j*ldb + k]  (bf16 in, fp32 accumulate).
 * out_mode 0: bf16 store, 1: fp32 store, 2: fp32 accumulate. The contraction used by the
 * entry points above, exported for tests (torch.mm in vocab_parallel_head.py:549-552). */
int areal_gemm_nt_bf16(const void* A, int64_t lda, const void* B, int64_t ldb, void* out,
                       int64_t ldo, int64_t M, int64_t N, int64_t K, int out_mode,
                       areal_stream_t stream);

/* dst (bf16) = src (fp32), n elements: the final cast of the weight gradient
 * (vocab_parallel_head.py:917-918). */
int areal_cast_f32_to_bf16(const float* src, void* dst, int64_t n, areal_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Logits-in label log-prob + entropy
 * replaces _gather_logprobs / _gather_logprobs_entropy and their chunked wrappers
 * (areal/utils/functional/vocab_parallel.py:16-30, :42-82, :564-651).
 * dtype: 0 = fp32 logits, 1 = bf16 logits; ld = row pitch in elements.
 * lse2 = log-sum-exp of logits/T in base-2 units (saved for backward).
 * ------------------------------------------------------------------------------------- */
int areal_logits_logprobs_entropy_fwd(const void* logits, int dtype, int64_t ld,
                                      const int64_t* labels, int64_t T, int64_t V,
                                      float inv_temperature, float* logprobs, float* entropy,
                                      float* lse2, areal_stream_t stream);

int areal_logits_logprobs_entropy_bwd(const void* logits, int dtype, int64_t ld,
                                      const int64_t* labels, int64_t T, int64_t V,
                                      float inv_temperature, const float* lse2,
                                      const float* entropy, const float* grad_logprobs,
                                      const float* grad_entropy, void* dlogits, int64_t ldd,
                                      areal_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Actor loss: PPO / GRPO clip (optionally dual clip, optionally GSPO sequence-level ratio) or
 * CISPO, with rejection sampling (IcePop ratio bounds, KPop binary KL, k1/k2/k3)
 * replaces ppo_actor_loss_fn (areal/utils/functional/functional.py:452-596), cispo_loss_fn
 * (:678-793), apply_rejection_sampling (:185-437), compute_binary_kl_divergence (:440-449) and
 * _compute_sequence_level_ratio_and_advantages (:56-149).
 * ------------------------------------------------------------------------------------- */
typedef struct areal_loss_config {
  int loss_kind;      /* -1: rejection sampling only, 0: PPO clip, 1: CISPO */
  float clip_lo;      /* (float)(1.0 - eps_clip) */
  float clip_hi;      /* (float)(1.0 + eps_clip_higher) */
  int has_c_clip;
  float c_clip;
  int seq_is;         /* importance_sampling_level == "sequence" */
  int rs_enabled;
  int rs_seq_level;   /* rejection_sampling.level == "sequence" */
  int rs_clamp;       /* rejection_sampling.action == "clamp" */
  int rs_metric;      /* 0 ratio, 1 kl_k1, 2 kl_k2, 3 kl_k3, 4 binary_kl */
  int rs_agg;         /* 0 sum, 1 mean, 2 max */
  float rs_upper;
  int rs_has_lower;
  float rs_lower;
} areal_loss_config;

size_t areal_actor_loss_workspace_bytes(int64_t n_tokens, int64_t n_seqs);

/* All per-token arrays have n_tokens elements (a packed 1-D batch or a flattened padded one).
 * Sequences: cu_seqlens [n_seqs+1] int32, or uniform_len > 0 for a padded [n_seqs, uniform_len]
 * batch; needed only for sequence-level options. cfg is a HOST pointer.
 * Outputs (each may be NULL): loss [1]; dlogprobs = d(sum of masked token losses)/dlogprobs
 * (divide by counters[1] for the loss gradient, see areal_actor_loss_grad); the per-token
 * statistics of the reference's stat dict; new_mask / behave_* of RejectionSamplingResult.
 * counters [8] double: loss_sum, n_valid (pre-rejection mask count), n_kept, n_filtered
 * (mask: rejected valid tokens; clamp: valid tokens whose weight changed), n_clip, n_dual_clip,
 * n_behave, loss. */
int areal_actor_loss(const float* logprobs, const float* proximal_logprobs,
                     const float* old_logprobs, const float* advantages,
                     const uint8_t* loss_mask, const int32_t* cu_seqlens, int64_t n_tokens,
                     int64_t n_seqs, int64_t uniform_len, const areal_loss_config* cfg,
                     float* loss, float* dlogprobs, float* stat_loss, float* stat_ratio,
                     float* stat_approx_kl, uint8_t* clip_mask, uint8_t* dual_clip_mask,
                     uint8_t* new_mask, float* behave_imp_weight, float* behave_approx_kl,
                     uint8_t* behave_mask, double* counters, void* workspace,
                     size_t workspace_bytes, areal_stream_t stream);

/* areal_actor_loss with the logging reductions folded into the token pass (replaces the clones
 * and the masked sum / min / max per logged tensor of stats_tracker,
 * areal/utils/stats_tracker.py:133-171, :455-560, as grpo_loss_fn uses them,
 * areal/trainer/ppo/actor.py:662-733). stats [17][4] double = {sum, count, min, max} of, in this
 * order: importance_weight, approx_kl, new_logp, old_logp, entropy, actor_loss, clip_ratio,
 * dual_clip_ratio, logp_diff, logp_abs_diff, behave_filtered_ratio (under the loss mask before
 * rejection), behave_imp_weight, behave_approx_kl (under the behave mask), clipped_new_logp,
 * clipped_old_logp (under the clip mask), extra0, extra1 (over every token; e.g. the vocabulary
 * min / max logits). min / max propagate NaN as torch.min / torch.max do; an empty denominator
 * gives count 0, min +inf, max -inf. entropy, extra0, extra1 are optional per-token inputs. Every
 * per-token output may be NULL: with only dlogprobs requested the call reads 17 (+4 entropy)
 * bytes per token and writes 4. */
size_t areal_actor_loss_stats_workspace_bytes(int64_t n_tokens, int64_t n_seqs);
int areal_actor_loss_stats(const float* logprobs, const float* proximal_logprobs,
                           const float* old_logprobs, const float* advantages,
                           const uint8_t* loss_mask, const int32_t* cu_seqlens, int64_t n_tokens,
                           int64_t n_seqs, int64_t uniform_len, const areal_loss_config* cfg,
                           const float* entropy, const float* extra0, const float* extra1,
                           float* loss, float* dlogprobs, float* stat_loss, float* stat_ratio,
                           float* stat_approx_kl, uint8_t* clip_mask, uint8_t* dual_clip_mask,
                           uint8_t* new_mask, float* behave_imp_weight, float* behave_approx_kl,
                           uint8_t* behave_mask, double* counters, double* stats, void* workspace,
                           size_t workspace_bytes, areal_stream_t stream);

/* areal_actor_loss without the workspace argument: the block partials and per-sequence
 * aggregates live in a static device array inside the library (about 1.7 MB per GPU, held until
 * the process ends), so nothing on the call path allocates. The first call on a device looks the
 * array's address up (hipGetSymbolAddress, once per device): make one call per device outside any
 * stream capture before a call is captured into a graph. It has no counterpart in the
 * reference; it is for callers that cannot allocate: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc. Call it with the stream's device current. At most
 * 65536 sequences (n_seqs beyond that: AREAL_ERR_UNSUPPORTED). All calls on one GPU share that
 * GPU's array: calls that overlap in time on one GPU race, calls on one stream do not. Outputs
 * are bit-identical to areal_actor_loss. */
int areal_actor_loss_static(const float* logprobs, const float* proximal_logprobs,
                            const float* old_logprobs, const float* advantages,
                            const uint8_t* loss_mask, const int32_t* cu_seqlens,
                            int64_t n_tokens, int64_t n_seqs, int64_t uniform_len,
                            const areal_loss_config* cfg, float* loss, float* dlogprobs,
                            float* stat_loss, float* stat_ratio, float* stat_approx_kl,
                            uint8_t* clip_mask, uint8_t* dual_clip_mask, uint8_t* new_mask,
                            float* behave_imp_weight, float* behave_approx_kl,
                            uint8_t* behave_mask, double* counters, areal_stream_t stream);

/* grad_logprobs[t] = dlogprobs[t] * upstream[0] / max(counters[1], 1): the backward of
 * `loss = sum(where(mask, pg, 0)) / loss_mask_count` (functional.py:571). */
int areal_actor_loss_grad(const float* dlogprobs, const float* upstream, const double* counters,
                          float* grad_logprobs, int64_t n_tokens, areal_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * SAPO policy loss, PPO critic loss, DPO sequence sums (same per-token layout as the actor loss)
 * replace sapo_loss_fn (areal/utils/functional/functional.py:599-675), ppo_critic_loss_fn
 * (:869-933) and the scatter-adds of dpo_pair_logratios (:796-841).
 * counters [8] double use the actor loss's layout ([0] loss sum, [1] denominator, [4] clipped
 * count, [7] loss), so areal_actor_loss_grad turns the d(loss sum) output into the gradient.
 * ------------------------------------------------------------------------------------- */
size_t areal_aux_loss_workspace_bytes(int64_t n_tokens, int64_t n_seqs);

/* seq_level != 0: geometric-mean ratio and mean advantage per sequence (functional.py:56-149;
 * cu_seqlens [n_seqs+1] or uniform_len > 0). Per-token outputs may be NULL.
 * stats (NULL allowed) [13][4] double = {sum, count, min, max} of what grpo_loss_fn logs for a
 * SAPO step (areal/trainer/ppo/actor.py:662-741), reduced inside the token pass instead of
 * written as [n_tokens] tensors: importance_weight, approx_kl, new_logp, old_logp, entropy,
 * actor_loss, logp_diff, logp_abs_diff, sapo_soft_gate, sapo_scaled_gate_pos,
 * sapo_scaled_gate_neg (under the loss mask), extra0, extra1 (every token). entropy, extra0,
 * extra1 [n_tokens] are optional inputs of that reduction (NULL: sum 0, min +inf, max -inf) and
 * are ignored without stats. */
int areal_sapo_loss(const float* logprobs, const float* old_logprobs, const float* advantages,
                    const uint8_t* loss_mask, const int32_t* cu_seqlens, int64_t n_tokens,
                    int64_t n_seqs, int64_t uniform_len, float tau_pos, float tau_neg,
                    int seq_level, float* loss, float* dlogprobs, float* stat_loss,
                    float* stat_ratio, float* stat_approx_kl, float* soft_gate, float* gate_pos,
                    float* gate_neg, double* counters, const float* entropy, const float* extra0,
                    const float* extra1, double* stats, void* workspace, size_t workspace_bytes,
                    areal_stream_t stream);

/* loss = mean over the mask (or over all n when loss_mask is NULL) of
 * max(l(value, target), l(old + clamp(value - old, +-eps), target)); l = mse or huber(10). */
int areal_critic_loss(const float* value, const float* old_value, const float* target_value,
                      const uint8_t* loss_mask, int64_t n, float value_eps_clip, int huber,
                      float* loss, float* dvalue, float* stat_loss, uint8_t* clip_mask,
                      double* counters, void* workspace, size_t workspace_bytes,
                      areal_stream_t stream);

/* M2PO second-moment mask (_apply_m2po_masking, areal/trainer/ppo/actor.py:933-1014): new_mask =
 * loss_mask minus the largest-m2 tokens (m2 = (old - prox)^2) that have to go for the mean m2 of
 * the rest to fall below m2_threshold; one token of a non-empty mask always stays. Found by a
 * radix select over the bit patterns of m2 instead of the reference's sort. */
size_t areal_m2po_mask_workspace_bytes(int64_t n_tokens);
int areal_m2po_mask(const float* old_logprobs, const float* proximal_logprobs,
                    const uint8_t* loss_mask, int64_t n_tokens, float m2_threshold,
                    uint8_t* new_mask, void* workspace, size_t workspace_bytes,
                    areal_stream_t stream);

/* Proximal log-prob approximation (compute_prox_logp_approximations,
 * areal/trainer/ppo/actor.py:768-848). versions [n] int64 (negative = prompt token). method 0
 * log-linear, 1 linear in probability space, 2 rollout. */
int areal_prox_logp_approx(const float* old_logprobs, const float* logprobs,
                           const int64_t* versions, int64_t n_tokens, int current_version,
                           int method, float* out, areal_stream_t stream);

/* Distillation terms of grpo_loss_fn (actor.py:629-658): value = sum(term) / max(count(mask), 1).
 * mode 0: term = (logprobs - teacher) * mask (joint KD + RL penalty); mode 1: term =
 * exp(logprobs - old) * (teacher - logprobs) * mask with the second factor held constant (pure
 * KD). dlogprobs = d(sum)/d logprobs; scale it with areal_actor_loss_grad. */
int areal_distill_terms(const float* logprobs, const float* old_logprobs,
                        const float* teacher_logprobs, const uint8_t* loss_mask, int64_t n_tokens,
                        int mode, float* value, float* dlogprobs, float* term, double* counters,
                        void* workspace, size_t workspace_bytes, areal_stream_t stream);

/* seq_sums [n_seqs][3] double = {sum policy log-probs, sum reference log-probs, count} over
 * shifted_mask[t] = loss_mask[t+1] inside each packed sequence (its last token excluded);
 * shifted_mask [n_tokens] is written for the backward. */
int areal_dpo_seq_logps(const float* logprobs, const float* ref_logprobs,
                        const uint8_t* loss_mask, const int32_t* cu_seqlens, int64_t n_tokens,
                        int64_t n_seqs, double* seq_sums, uint8_t* shifted_mask,
                        areal_stream_t stream);

/* grad_logprobs[t] = shifted_mask[t] * grad_seq[sequence of t]. */
int areal_dpo_seq_logps_grad(const double* grad_seq, const uint8_t* shifted_mask,
                             const int32_t* cu_seqlens, int64_t n_tokens, int64_t n_seqs,
                             float* grad_logprobs, areal_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * GAE over packed sequences
 * replaces _compute_token_level_gae (areal/trainer/ppo/gae.py:10-36); per-sequence lambda as
 * produced by areal/trainer/ppo/lambda_fn.py:50-112.
 * ------------------------------------------------------------------------------------- */
size_t areal_gae_workspace_bytes(int64_t n_tokens);

int areal_gae_packed(const float* rewards, const float* values, const float* loss_mask,
                     const int32_t* cu_seqlens, const uint8_t* no_eos, const float* lambda_seq,
                     int64_t n_tokens, int64_t n_seqs, int64_t uniform_len, float discount,
                     float gae_lambda, float* advantages, float* returns, void* workspace,
                     size_t workspace_bytes, areal_stream_t stream);

/* areal_gae_packed on a padded [n_seqs, uniform_len] batch with rows of at least 2048 tokens
 * (AREAL_ERR_UNSUPPORTED otherwise), which also leaves per row, in row_stats [5][n_seqs] fp64, the
 * sums of m, x m, m^2, m^2 x, m^2 x^2 (x = the advantage written, m = loss_mask): the statistics
 * pass of the advantage normalisation that follows in compute_advantages
 * (areal/trainer/ppo/actor.py:344-350: adv_norm(advantages, loss_mask)), at no extra traffic. */
int areal_gae_padded_row_stats(const float* rewards, const float* values, const float* loss_mask,
                               const uint8_t* no_eos, const float* lambda_seq, int64_t n_seqs,
                               int64_t uniform_len, float discount, float gae_lambda,
                               float* advantages, float* returns, double* row_stats,
                               areal_stream_t stream);

/* areal_gae_packed on packed sequences (cu_seqlens) that also leaves the statistics pass of a
 * group normalisation of the advantages under loss_mask (areal/trainer/ppo/actor.py:344-350 on
 * the packed layout): groups are runs of whole sequences, group_offsets [n_groups + 1] (int64,
 * device) their token offsets from 0 to n_tokens. segment_stats (fp64,
 * areal_gae_segment_stats_bytes(n_tokens, n_groups) bytes) receives the five sums of
 * areal_gae_padded_row_stats per (2048-token tile, group) segment, for
 * areal_group_norm_from_segment_stats. One launch. AREAL_ERR_UNSUPPORTED when sequences average
 * more than 16384 tokens or groups fewer than 256: run areal_gae_packed and areal_group_norm. */
size_t areal_gae_segment_stats_bytes(int64_t n_tokens, int64_t n_groups);
int areal_gae_packed_group_stats(const float* rewards, const float* values, const float* loss_mask,
                                 const int32_t* cu_seqlens, const uint8_t* no_eos,
                                 const float* lambda_seq, int64_t n_tokens, int64_t n_seqs,
                                 float discount, float gae_lambda, const int64_t* group_offsets,
                                 int64_t n_groups, float* advantages, float* returns,
                                 double* segment_stats, size_t segment_stats_bytes,
                                 areal_stream_t stream);

/* Turn-level GAE (areal/trainer/ppo/gae.py:82-163) on padded [bs, max_seqlen] tensors: every
 * generated turn is one timestep. turn_ids int32 (-1 in prompt / tool gaps; non-decreasing over
 * the active tokens of a row), loss_mask fp32 (nonzero = active). *status (device int, zeroed
 * by the caller) receives a bit mask of malformed ids at active tokens: 1 negative, 2 not
 * smaller than max_seqlen, 4 decreasing (the conditions _validate_turn_ids asserts, :39-79). */
size_t areal_turn_gae_workspace_bytes(int64_t bs, int64_t max_seqlen);
int areal_turn_gae(const float* rewards, const float* values, const float* loss_mask,
                   const int32_t* turn_ids, const uint8_t* no_eos, const float* lambda_seq,
                   int64_t bs, int64_t max_seqlen, float discount, float gae_lambda,
                   float* advantages, float* returns, int* status, void* workspace,
                   size_t workspace_bytes, areal_stream_t stream);

/* Per-row lengths for per-sample lambda functions (_build_gae_lambda_context,
 * areal/trainer/ppo/gae.py:166-205): active tokens, and distinct turn ids among them (turn_ids
 * may be NULL: turn counts 0). status as in areal_turn_gae. */
int areal_gae_lambda_context(const float* loss_mask, const int32_t* turn_ids, int64_t bs,
                             int64_t max_seqlen, int64_t* token_lengths, int64_t* turn_counts,
                             int* status, areal_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Normalisation
 * replaces Normalization.__call__ / _compute_mean / _compute_std
 * (areal/utils/data.py:1432-1637) and masked_normalization
 * (areal/utils/functional/functional.py:16-53). Levels: 0 none, 1 batch, 2 group.
 * ------------------------------------------------------------------------------------- */
size_t areal_group_norm_workspace_bytes(int64_t n_groups, int64_t max_group_len);

int areal_group_norm(const float* x, const float* mask, int64_t n, const int64_t* group_offsets,
                     const int64_t* group_rows, int64_t n_groups, int64_t max_group_len,
                     int tail_group, int mean_level, int std_level, int leave_one_out,
                     int unbiased, double eps, float* out, void* workspace,
                     size_t workspace_bytes, areal_stream_t stream);

/* The apply pass of areal_group_norm alone (one launch), for a [n_rows, row_len] array whose
 * per-row sums are already known (row_stats as areal_gae_padded_row_stats leaves them). Groups
 * are runs of whole rows. Only for level combinations that need no second statistics pass: no
 * leave-one-out mean, and not a group-level mean under a batch-level deviation
 * (AREAL_ERR_UNSUPPORTED). Same arithmetic as Normalization.__call__
 * (areal/utils/data.py:1382-1637) with the sum of squared deviations evaluated in fp64 from the
 * sums. */
int areal_group_norm_from_row_stats(const float* x, const float* mask, int64_t n_rows, int64_t row_len,
                                    const int64_t* group_offsets, const int64_t* group_rows,
                                    int64_t n_groups, int64_t max_group_len, int tail_group,
                                    int mean_level, int std_level, int unbiased, double eps,
                                    const double* row_stats, float* out, areal_stream_t stream);

/* The same apply pass on a packed array of n elements whose segment sums
 * areal_gae_packed_group_stats left (same n and group_offsets): one launch, same restrictions. */
int areal_group_norm_from_segment_stats(const float* x, const float* mask, int64_t n,
                                        const int64_t* group_offsets, const int64_t* group_rows,
                                        int64_t n_groups, int64_t max_group_len, int tail_group,
                                        int mean_level, int std_level, int unbiased, double eps,
                                        const double* segment_stats, float* out,
                                        areal_stream_t stream);

size_t areal_masked_norm_workspace_bytes(int64_t n);

int areal_masked_norm(const float* x, const float* mask, int64_t n, int unbiased, double eps,
                      float* out, void* workspace, size_t workspace_bytes, areal_stream_t stream);

/* Reward shaping in front of GAE (PPOActor.compute_advantages, areal/trainer/ppo/actor.py:224-283)
 * on a padded [bs, L] batch, one pass instead of the reference's elementwise tensor ops: rolled
 * float loss mask, masked old log-probs, KL rewards by the k1/k2/k3 estimator
 * (areal/utils/data.py:1662-1698; estimator = 1, 2, 3), their copy zeroed at the last token, the
 * outcome reward placed at max(seqlen - 2, 0), and their sum; per row the sequence length (sum of
 * attn_mask) and whether the row is full (no EOS). loss_mask / attn_mask are bytes; ref_logp,
 * gkl_out, outcome_out may be NULL. roll_logp = 0 takes logp as already aligned (the
 * recompute_logprob branch, actor.py:246-253) and then old_out may be logp itself; ref_in_place
 * writes the masked ref_logp back, as the reference's in-place `ref_logp *= loss_mask` does. */
int areal_advantage_prep(const uint8_t* loss_mask, const uint8_t* attn_mask, const float* logp,
                         float* ref_logp, const float* reward_score, int64_t bs, int64_t L,
                         int roll_logp, int estimator, int apply_clamp, int mask_no_eos_with_zero,
                         int ref_in_place, float kl_ctl, float* lm_out, float* old_out,
                         float* kl_out, float* gkl_out, float* outcome_out, float* tot_out,
                         int64_t* seqlens_out, uint8_t* no_eos_out, areal_stream_t stream);

/* masked_normalization with dim = the trailing dimensions (areal/utils/functional/functional.py:16-53,
 * the `dim` argument): x, mask (NULL allowed) and out are [rows, cols]; every row is whitened with
 * its own masked mean and variance. */
int areal_masked_norm_rows(const float* x, const float* mask, int64_t rows, int64_t cols,
                           int unbiased, double eps, float* out, areal_stream_t stream);

/* ---------------------------------------------------------------------------------------
 * Packing / padding by cu_seqlens and masked logging statistics (the steps either side of the
 * loss). Replace the per-sequence Python loops of pack_tensor_dict (areal/utils/data.py:496-545),
 * pad_packed_tensor_dict (:822-982), unpack_sequence + reorder_list +
 * pad_and_stack_tensors_along_first_dim as composed by reorder_and_pad_outputs
 * (areal/engine/core/train_engine.py:110-144), and the per-tensor torch.where(...).sum() / min /
 * max of stats_tracker (areal/utils/stats_tracker.py:455-560).
 * elem_bytes = bytes of one token's trailing dimensions; fill = up to 16 bytes repeated over an
 * element (NULL = zeros).
 * ------------------------------------------------------------------------------------- */
int areal_seqlens_from_mask(const uint8_t* attention_mask, int64_t B, int64_t S, int32_t* lens,
                            int32_t* cu_seqlens, int32_t* max_len, areal_stream_t stream);
int areal_pack_padded(const void* padded, void* packed, const int32_t* cu_seqlens, int64_t B,
                      int64_t S, int64_t elem_bytes, int64_t total, areal_stream_t stream);
/* The tensors of one batch (pack_tensor_dict's loop over the dict, data.py:519-543) in one launch:
 * padded / packed / elem_bytes are HOST arrays of n_tensors (at most 8) device pointers, resp.
 * element sizes. */
int areal_pack_padded_multi(const void* const* padded, void* const* packed,
                            const int64_t* elem_bytes, int n_tensors, const int32_t* cu_seqlens,
                            int64_t B, int64_t S, int64_t total, areal_stream_t stream);
int areal_unpack_to_padded(const void* packed, void* padded, const int32_t* cu_seqlens,
                           const int32_t* row_seq, int64_t B, int64_t S, int64_t elem_bytes,
                           const void* fill, int fill_bytes, areal_stream_t stream);
/* Sequence s moves from cu_old to cu_new (new length >= old, tail filled); sequences of cu_new
 * beyond n_old are all fill. position_ids != 0 (int64 elements): src NULL writes 0..len-1 per
 * new sequence, otherwise the filled parts count 0, 1, 2, ... */
int areal_realign_packed(const void* src, void* dst, const int32_t* cu_old, int64_t n_old,
                         const int32_t* cu_new, int64_t n_new, int64_t elem_bytes,
                         const void* fill, int fill_bytes, int position_ids, int64_t total_new,
                         areal_stream_t stream);
size_t areal_masked_stats_workspace_bytes(int K);
/* out [K][4] double = {sum, count, min, max} of values[k] where masks[k] != 0 (NULL mask: all).
 * values / masks are HOST arrays of K <= 32 device pointers. */
int areal_masked_stats(const float* const* values, const uint8_t* const* masks, int K, int64_t n,
                       double* out, void* workspace, size_t workspace_bytes,
                       areal_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* AREAL_HIP_H */
