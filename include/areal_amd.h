/*
 * areal_amd.h -- C ABI of the MI355X (gfx950) kernels behind AReaL's PPO/GRPO
 * log-prob / entropy / actor-loss path.
 *
 * Every entry point takes plain device pointers and sizes, enqueues its work on
 * the HIP stream it is given (hipStream_t passed as void*; NULL = the default
 * stream), allocates nothing, and never synchronises the device.  The return
 * value is an aa_status; a non-zero value means nothing was enqueued.
 *
 * Layout conventions (the reference's "packed 1-D" layout):
 *   logits      [T, V]  row-major, element (t, j) at logits[t * row_stride + j]
 *   labels      [T]     int64, already rolled by the caller
 *   cu_seqlens  [B+1]   int32, cu_seqlens[i] = first token of sequence i
 *   per-token   [T]     float32 unless stated, masks are one byte per token
 *
 * Reference citations are relative to the AReaL source tree.
 */
#ifndef AREAL_AMD_H
#define AREAL_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  AA_OK = 0,
  AA_ERR_INVALID_ARGUMENT = 1,
  AA_ERR_UNSUPPORTED = 2,
  AA_ERR_LAUNCH = 3
} aa_status;

/* element type of logits / hidden / weight buffers */
typedef enum { AA_BF16 = 0, AA_F16 = 1, AA_F32 = 2 } aa_dtype;

/* rejection-sampling switches; mirror RejectionSamplingConfig
 * (areal/api/cli_args.py:1223-1385) */
typedef enum { AA_RS_LEVEL_TOKEN = 0, AA_RS_LEVEL_SEQUENCE = 1 } aa_rs_level;
typedef enum { AA_RS_ACTION_MASK = 0, AA_RS_ACTION_CLAMP = 1 } aa_rs_action;
typedef enum { AA_RS_RATIO = 0, AA_RS_KL_K1 = 1, AA_RS_KL_K2 = 2, AA_RS_KL_K3 = 3 } aa_rs_metric;
typedef enum { AA_RS_AGG_SUM = 0, AA_RS_AGG_MEAN = 1, AA_RS_AGG_MAX = 2 } aa_rs_agg;

/* Which per-token loss the fused entry points put on the log-probs:
 *   AA_LOSS_PPO  the clipped surrogate of ppo_actor_loss_fn
 *                (areal/utils/functional/functional.py:516-542), divided by
 *                max(*n_valid, 1);
 *   AA_LOSS_NLL  the supervised loss of compute_packed_sft_loss
 *                (areal/trainer/sft/lm_engine.py:93-96): -logp on the selected
 *                tokens, divided by (*n_valid + 1e-5).  stat_loss = -logp on
 *                the selected tokens and 0 elsewhere, ratio = 0, flags = 0; prox_logp, adv and behave_w are not
 *                used and may be NULL;
 *   AA_LOSS_SAPO the token-level loss of sapo_loss_fn
 *                (areal/utils/functional/functional.py:589-622): with r =
 *                exp(logp - prox_logp) (the caller passes the behaviour
 *                log-probs there: SAPO has no proximal policy), -adv * 4 / tau *
 *                sigmoid(tau (r - 1)) with tau = sapo_tau_pos where adv > 0 and
 *                sapo_tau_neg elsewhere, divided by max(*n_valid, 1).  ratio
 *                and stat_loss are those of the reference at every token
 *                (the ratio is not zeroed at masked tokens), flags = 0;
 *                has_behave_weight must be 0. */
typedef enum { AA_LOSS_PPO = 0, AA_LOSS_NLL = 1, AA_LOSS_SAPO = 2 } aa_loss_kind;

/* Clipped-surrogate parameters of ppo_actor_loss_fn
 * (areal/utils/functional/functional.py:516-532). */
typedef struct {
  float clip_lo;       /* 1 - eps_clip                                   */
  float clip_hi;       /* 1 + (eps_clip_higher or eps_clip)              */
  float c_clip;        /* dual-clip factor, used only if has_c_clip != 0 */
  int32_t has_c_clip;
  int32_t has_behave_weight; /* multiply the loss by behave_w (rejection sampling on) */
  int32_t loss_kind;   /* aa_loss_kind; aa_ppo_loss accepts AA_LOSS_PPO only */
  float sapo_tau_pos;  /* AA_LOSS_SAPO: gate temperatures, both > 0      */
  float sapo_tau_neg;
} aa_ppo_params;

/* Library version (major * 10000 + minor * 100 + patch). */
int aa_version(void);

/* Text for an aa_status value (static storage). */
const char* aa_status_string(int status);

/* ------------------------------------------------------------------ */
/* Logits path                                                         */
/* ------------------------------------------------------------------ */

/*
 * Forward of gather_logprobs / gather_logprobs_entropy
 * (areal/utils/functional/vocab_parallel.py:15-29, 401-469): one streaming
 * pass per row, fp32 online softmax.
 *   logp[t]    = z[label] - logsumexp(z),  z = logits[t, :] / temperature
 *   entropy[t] = logsumexp(z) - sum_j softmax(z)_j * z_j          (nullable)
 *   row_lse[t] = logsumexp(z)     row_ez[t] = sum_j softmax(z)_j z_j
 *                (nullable; what aa_logits_bwd needs)
 *   vmax / vmin = max / min of the raw row (nullable; replaces the two extra
 *                passes of FSDPEngine._get_vocab_min_max_logits,
 *                areal/engine/fsdp_engine.py:1893-1906)
 * A label outside [0, V) yields logp = NaN and never faults.
 */
int aa_logits_fwd(const void* logits, int dtype, int64_t T, int64_t V,
                  int64_t row_stride, const int64_t* labels,
                  float inv_temperature, float* logp, float* entropy,
                  float* row_lse, float* row_ez, float* vmax, float* vmin,
                  void* stream);

/*
 * Backward of the same op (autograd of vocab_parallel.py:15-29; closed form
 * as in vocab_parallel.py:339-370):
 *   dlogits[t, j] = inv_temperature * ( g_logp[t] * (1[j == label] - p_j)
 *                                     + g_entropy[t] * p_j * (row_ez[t] - z_j) )
 * g_entropy may be NULL (treated as zero).  dlogits has the dtype and row
 * stride of logits.  Rows with t >= T_active (the batch padding the caller
 * trims after the op, fsdp_engine.py:2027-2031) are written as zeros.
 * dlogits may be the logits array itself (every element is read before it is
 * written, by the same thread); any other overlap is not allowed.
 */
int aa_logits_bwd(const void* logits, int dtype, int64_t T, int64_t V,
                  int64_t row_stride, const int64_t* labels,
                  float inv_temperature, const float* row_lse,
                  const float* row_ez, const float* g_logp,
                  const float* g_entropy, int64_t T_active, void* dlogits,
                  void* stream);

/*
 * Fused forward + token-level PPO loss + backward for one micro-batch
 * (vocab_parallel.py:23-29 -> functional.py:429-559 with
 * importance_sampling_level="token" -> autograd), one launch:
 * each row is read once, and d(loss)/d(logits) is written once.
 *
 * Per-token inputs [T_active]: prox_logp, adv, mask_eff (uint8, the mask after
 * rejection sampling), behave_w (nullable unless params->has_behave_weight);
 * with T_active == 0 they and the [T_active] outputs may all be NULL.
 * n_valid: device pointer to the int32 count of non-zero entries of the
 *   ORIGINAL loss mask (functional.py:483); the loss is divided by
 *   max(*n_valid, 1).
 * grad_scale: device pointer to a float the gradient is multiplied by (the
 *   engine's local_weight / total_loss_weight * multiplier,
 *   fsdp_engine.py:2045); NULL = 1.
 * Outputs [T]: logp, entropy (nullable), vmax, vmin (nullable);
 * outputs [T_active]: stat_loss (per-token surrogate times behave_w, before
 *   masking), ratio, flags (bit0 = clip_mask & mask_eff, bit1 =
 *   dual_clip_mask & mask_eff); dlogits [T, V] in the dtype of logits (rows
 *   >= T_active are zeros).  The scalar loss is finished by aa_masked_sum.
 * dlogits may be the logits array itself (the gradient then takes the place
 *   of the logits, which halves the memory of the step; no counterpart in the
 *   reference, whose autograd allocates the gradient): a row belongs to one
 *   workgroup, and every kernel behind this entry point reads an element for
 *   the last time before it writes it.  Any other overlap of the two arrays
 *   is not allowed.
 * work: NULL, or two int32 words of device memory that are zero on entry; the
 *   kernel hands rows to compute units through them (faster than a fixed
 *   assignment) and leaves them zero on exit, so one zeroed buffer serves
 *   every launch on a stream.  Launches that may run concurrently need
 *   separate buffers.
 * Layout: any V, any row_stride >= V, logits and dlogits at any address that
 *   their element size divides.  16-bit rows of 16 385 to 262 136 values are
 *   read once and held in registers whatever their alignment, provided that
 *   logits and dlogits start at the same offset inside a 16-byte piece of
 *   memory (both on a 16-byte boundary, the usual case, or both k bytes past
 *   one); otherwise the rows that are not on 16-byte boundaries are read
 *   twice.
 * AA_F32 logits with V % 8 == 0 and more than 114 688 values per row: the row
 *   is kept on the chip between its read and the write of its gradient in 24
 *   bits per value (a 608 KB row of V = 151 936 does not fit the register file
 *   in fp32).  logp, entropy, vmax and vmin are computed from the fp32 values;
 *   the softmax probabilities behind dlogits carry a relative error of at
 *   most |x_j| * inv_temperature * 2^-16 (2e-4 at 13), ten times finer than
 *   the rounding of a bf16 gradient row.  Shorter fp32 rows are kept exactly.
 */
int aa_logits_ppo_fused(const void* logits, int dtype, int64_t T, int64_t V,
                        int64_t row_stride, const int64_t* labels,
                        float inv_temperature, int64_t T_active,
                        const float* prox_logp, const float* adv,
                        const uint8_t* mask_eff, const float* behave_w,
                        const aa_ppo_params* params, const int32_t* n_valid,
                        const float* grad_scale, float* logp, float* entropy,
                        float* vmax, float* vmin, float* stat_loss,
                        float* ratio, uint8_t* flags, void* dlogits,
                        int32_t* work, void* stream);

/*
 * The reduction step of the vocabulary-parallel op
 * (areal/utils/functional/vocab_parallel.py:84-372), for n_shards slices
 * [T, V_i] of one [T, V] logits tensor that each went through aa_logits_fwd
 * with the labels shifted into the slice (a label outside it gives NaN there):
 *   shard_lse, shard_ez, shard_logp: [n_shards, T], the row_lse, row_ez and
 *   logp outputs of those calls;
 *   row_lse = logsumexp_i shard_lse_i,  row_ez = sum_i exp(shard_lse_i -
 *   row_lse) * shard_ez_i,  logp = shard_logp_i + shard_lse_i - row_lse for the
 *   shard that holds the label (NaN if none does),  entropy = row_lse - row_ez.
 * entropy, row_lse, row_ez may be NULL.  The backward of a slice is
 * aa_logits_bwd on that slice with the shifted labels and the combined
 * row_lse / row_ez.  Across GPUs the three [T] vectors per rank are what one
 * exchange carries; the exchange itself is not part of this library.
 */
int aa_vocab_partials_combine(const float* shard_lse, const float* shard_ez,
                              const float* shard_logp, int n_shards, int64_t T,
                              float* logp, float* entropy, float* row_lse,
                              float* row_ez, void* stream);

/*
 * Log-probs for arbitrary (row, label) pairs, the transitions of a packed
 * prefix tree (areal/models/tree_attn/functional.py:160-203, 206-316), where a
 * row may predict several tokens that sit elsewhere in the packed tensor:
 *   logp[k] = logits[rows[k], labels[k]] * inv_temperature - row_lse[rows[k]]
 *   entropy[k] = row_entropy[rows[k]]                               (nullable)
 * row_lse / row_entropy come from one aa_logits_fwd pass over the rows.
 * A row or label out of range gives NaN.
 */
int aa_logits_pairs_fwd(const void* logits, int dtype, int64_t T, int64_t V,
                        int64_t row_stride, const int64_t* rows,
                        const int64_t* labels, int64_t K,
                        float inv_temperature, const float* row_lse,
                        const float* row_entropy, float* logp, float* entropy,
                        void* stream);

/*
 * The one-hot part of the backward of aa_logits_pairs_fwd:
 *   dlogits[rows[k], labels[k]] += g[k] * inv_temperature
 * (the softmax part is aa_logits_bwd with the per-row sums of g and a label of
 * -1).  The pairs must be distinct: the update is a plain read-modify-write.
 */
int aa_logits_pairs_scatter(void* dlogits, int dtype, int64_t T, int64_t V,
                            int64_t row_stride, const int64_t* rows,
                            const int64_t* labels, int64_t K, const float* g,
                            float inv_temperature, void* stream);

/* ------------------------------------------------------------------ */
/* Per-token PPO pieces                                                */
/* ------------------------------------------------------------------ */

/*
 * apply_rejection_sampling (functional.py:185-426) on packed tokens.
 * Segments come from cu_seqlens [B+1], or, when cu_seqlens is NULL, are B
 * equal-length rows of n / B tokens (the reference's 2-D padded layout).
 *   mask_in  uint8 [n]  (non-zero = valid)
 *   mask_out uint8 [n]  updated mask (action mask) or a copy (action clamp)
 *   behave_w float [n]  importance weight, zero where mask_out is zero
 *   counts   int32 [3]  {non-zero entries of mask_in, filtered-or-clamped
 *                        valid tokens, unused}; written, not accumulated
 * lower is ignored unless has_lower != 0.
 */
int aa_rejection_sampling(const float* prox_logp, const float* old_logp,
                          const uint8_t* mask_in, int64_t n,
                          const int32_t* cu_seqlens, int64_t B, int level,
                          int action, int metric, int agg, float upper,
                          float lower, int has_lower, uint8_t* mask_out,
                          float* behave_w, int32_t* counts, void* stream);

/* counts[0] = number of non-zero bytes of mask[0..n) (functional.py:483). */
int aa_count_nonzero_u8(const uint8_t* mask, int64_t n, int32_t* count,
                        void* stream);

/*
 * ppo_actor_loss_fn given log-probs (functional.py:429-559), both
 * importance-sampling levels, forward and closed-form backward in one call.
 *   sequence_level != 0 selects the GSPO branch (functional.py:56-149), which
 *   needs segments (cu_seqlens / B as in aa_rejection_sampling).
 * Outputs [n]: stat_loss, ratio, flags (as in aa_logits_ppo_fused),
 *   g_logp = d(loss)/d(logp) with loss = sum(mask_eff ? stat_loss : 0) /
 *   max(*n_valid, 1).  The scalar loss is finished by aa_masked_sum.
 */
int aa_ppo_loss(const float* logp, const float* prox_logp, const float* adv,
                const uint8_t* mask_eff, const float* behave_w, int64_t n,
                const int32_t* cu_seqlens, int64_t B, int sequence_level,
                const aa_ppo_params* params, const int32_t* n_valid,
                float* stat_loss, float* ratio, uint8_t* flags, float* g_logp,
                void* stream);

/*
 * The derived entries of the stat dict of ppo_actor_loss_fn
 * (functional.py:505-558), which the reference forms with one small launch
 * each, in one launch:
 *   approx_kl = logp - prox_logp;  clip_mask, dual_clip_mask = bit 0 and bit 1
 *   of flags (bytes 0 / 1);  and, when behave_mask is given (rejection
 *   sampling), behave_mask = behave_w > 0 && mask_eff != 0 and
 *   behave_approx_kl = behave_mask ? prox_logp - old_logp : 0.
 * behave_mask and behave_approx_kl are both NULL or both given (then old_logp,
 * behave_w and mask_eff are required).
 */
int aa_ppo_stat_outputs(const float* logp, const float* prox_logp,
                        const float* old_logp, const uint8_t* flags,
                        const float* behave_w, const uint8_t* mask_eff,
                        int64_t n, float* approx_kl, uint8_t* clip_mask,
                        uint8_t* dual_clip_mask, uint8_t* behave_mask,
                        float* behave_approx_kl, void* stream);

/*
 * out[0] = scale * sum_{i<n, mask[i] != 0} values[i] / max(*n_valid, 1)
 * (functional.py:542), accumulated in a fixed order so that repeated calls are
 * bit-identical.  n_valid may be NULL (divide by 1); scale may be NULL (1);
 * mask may be NULL (every element counts).
 */
int aa_masked_sum(const float* values, const uint8_t* mask, int64_t n,
                  const int32_t* n_valid, const float* scale, float* out,
                  void* stream);

/* data[i] *= *factor for i < n (dtype as aa_dtype); a no-op when *factor == 1. */
int aa_scale_inplace(void* data, int dtype, int64_t n, const float* factor,
                     void* stream);

/*
 * The same for T rows of V elements that start row_stride >= V elements apart
 * (the upstream factor of loss.backward() on a gradient that lies in a slice
 * of a wider array: what lies between the rows is not touched).
 */
int aa_scale_rows_inplace(void* data, int dtype, int64_t T, int64_t V,
                          int64_t row_stride, const float* factor,
                          void* stream);

/* ------------------------------------------------------------------ */
/* Sibling losses and actor-side token filters                            */
/* ------------------------------------------------------------------ */

/*
 * sapo_loss_fn (functional.py:562-638): asymmetric sigmoid gates in place of
 * clipping, forward and closed-form backward.  ratio = exp(logp - old_logp)
 * (token level, unmasked) or the per-sequence geometric mean
 * (sequence_level != 0, segments as in aa_ppo_loss).
 * Outputs [n]: stat_loss = -soft_gate * adv, ratio, g_logp; gates [3, n] =
 * {soft gate, scaled positive gate, scaled negative gate}.  The scalar loss
 * is aa_masked_sum(stat_loss, mask, n_valid).
 */
int aa_sapo_loss(const float* logp, const float* old_logp, const float* adv,
                 const uint8_t* mask, int64_t n, const int32_t* cu_seqlens,
                 int64_t B, int sequence_level, float tau_pos, float tau_neg,
                 const int32_t* n_valid, float* stat_loss, float* ratio,
                 float* gates, float* g_logp, void* stream);

/*
 * ppo_critic_loss_fn (functional.py:704-778): clipped value loss, forward and
 * closed-form backward (torch.max ties split in half, clamp passes gradient
 * on the closed interval).  loss_type 0 = mse, 1 = huber (delta 10).
 * mask may be NULL (plain mean); *n_valid is the divisor (count of non-zero
 * mask bytes, or n) and is NOT floored at 1, as in the reference.
 * Outputs [n]: stat_loss = max(original, clipped), clip_mask bytes, g_value.
 */
int aa_critic_loss(const float* value, const float* old_value,
                   const float* target_value, const uint8_t* mask, int64_t n,
                   float value_eps_clip, int loss_type, const int32_t* n_valid,
                   float* stat_loss, uint8_t* clip_mask, float* g_value,
                   void* stream);

/*
 * compute_prox_logp_approximations (areal/trainer/ppo/actor.py:604-684):
 * method 0 = loglinear, 1 = linear (probability space), 2 = rollout.
 * versions: per-token policy version, int32, negative for prompt tokens.
 */
int aa_prox_logp_approx(const float* old_logp, const float* logp,
                        const int32_t* versions, int64_t n,
                        int current_version, int method, float* out,
                        void* stream);

/*
 * KLEstimator (areal/utils/data.py:1598-1656) per element, d = logp -
 * logp_base: estimator 0 (k1) = d, 1 (k2) = d^2 / 2, 2 (k3) = exp(-d) - 1 + d;
 * apply_clamp != 0 clamps the result to [-10, 10].
 */
int aa_kl_estimate(const float* logp, const float* logp_base, int64_t n,
                   int estimator, int apply_clamp, float* out, void* stream);

/* Bytes of 256-byte aligned scratch aa_masked_normalization needs. */
int64_t aa_masked_normalization_scratch_bytes(int64_t rows, int64_t cols);

/*
 * masked_normalization (areal/utils/functional/functional.py:16-53) over the
 * last axis of an [rows, cols] view (the reference's `dim` axes brought to the
 * back; dim=None is rows = 1).  mask float32 of the same shape or NULL.  With
 * v = x * mask, F = sum(mask) (cols when mask is NULL), per row in float64:
 *   mean = sum(v) / F, var = sum(v^2) / F - mean^2, var *= F / (F - 1) when
 *   unbiased != 0; out = (float)((v - mean) / (sqrt(var) + eps)).
 * Masked positions are whitened as zeros, as in the reference.  Sums are
 * always float64 (the reference's high_precision=True), in a fixed order.
 * The reference's all-reduce over a process group is not part of this call.
 */
int aa_masked_normalization(const float* x, const float* mask, int64_t rows,
                            int64_t cols, int unbiased, double eps, float* out,
                            void* scratch, int64_t scratch_bytes, void* stream);

/*
 * reward_overlong_penalty (functional.py:782-803), in place on rewards [bs]:
 *   len_b = (long) sum(loss_mask[b, :])           loss_mask [bs, L] float32
 *   rewards[b] += min(-(len_b - (max_response_length - overlong_tokens))
 *                     / overlong_tokens * overlong_penalty_factor, 0)
 */
int aa_overlong_penalty(float* rewards, const float* loss_mask, int64_t bs,
                        int64_t L, int overlong_tokens,
                        float overlong_penalty_factor,
                        int64_t max_response_length, void* stream);

/*
 * Per-token terms of the joint-distillation branch of grpo_loss_fn
 * (trainer/ppo/actor.py:482-511), with mask the bool loss mask as bytes:
 *   pure_distillation != 0 (rl_loss_weight == 0, :493-503):
 *     term = exp(logp - old_logp) * (teacher_logp - logp) * mask, the reward
 *     (teacher_logp - logp) detached, so dterm = d term / d logp = term;
 *     loss = -distill_loss_weight * sum(term) / max(sum(mask), 1),
 *     rkl statistic = -term.
 *   otherwise (:504-511): term = (logp - teacher_logp) * mask, dterm = mask;
 *     loss = rl_loss_weight * loss + distill_loss_weight * sum(term) /
 *     max(sum(mask), 1), rkl statistic = term.
 * The sums are finished by aa_masked_sum.  old_logp may be NULL in the second
 * form.
 */
int aa_kd_terms(const float* logp, const float* old_logp,
                const float* teacher_logp, const uint8_t* mask, int64_t n,
                int pure_distillation, float* term, float* dterm,
                void* stream);

/*
 * compute_packed_sft_loss (areal/trainer/sft/lm_engine.py:81-131) given
 * log-probs: with m the loss mask as bytes and n = *n_valid (device, the
 * number of non-zero mask bytes, aa_count_nonzero_u8),
 *   loss[0]      = -scale * sum_t (m ? logp[t] : 0) / (n + 1e-5)
 *   g_logp[t]    = d loss / d logp[t] = m ? -scale / (n + 1e-5) : 0  (nullable)
 *   stat_loss[t] = -(m ? logp[t] : 0), what the reference logs per token
 *                  (nullable)
 * and per sequence b of cu_seqlens [n_seqs + 1] (int32, device; the Python
 * loop with one read-back per sequence at :101-112):
 *   seq_count[b] = selected tokens of the sequence,
 *   seq_logp[b]  = mean of their log-probs in fp64, 0 when there is none,
 *   seq_ppl[b]   = (float)exp(-seq_logp[b])                          (nullable)
 * seq_logp and seq_count have n_seqs + 1 entries; the last holds the sum and
 * the number of the selected tokens outside every sequence.  cu_seqlens may be
 * NULL with n_seqs == 0.  scale: device float, NULL = 1.  Sums are fp64 in a
 * fixed order.
 */
int aa_sft_loss(const float* logp, const uint8_t* mask, int64_t T,
                const int32_t* cu_seqlens, int64_t n_seqs,
                const int32_t* n_valid, const float* scale, float* loss,
                float* g_logp, float* stat_loss, double* seq_logp,
                int32_t* seq_count, float* seq_ppl, void* stream);

/*
 * Direct preference optimisation over a packed batch whose sequences are
 * interleaved [chosen_0, rejected_0, chosen_1, rejected_1, ...].
 *
 * aa_dpo_seq_sums: the per-sequence aggregation of dpo_pair_logratios
 * (areal/utils/functional/functional.py:641-687) before the pairing view.
 * loss_mask [T] bytes, cu_seqlens [n_seqs + 1] int32 on the device.  With
 * shifted[t] = loss_mask[t + 1] inside a sequence and 0 at its last position:
 *   policy_sums[s]     = sum_t (double)(logp[t] * shifted[t])
 *   ref_sums[s]        = sum_t (double)(ref_logp[t] * shifted[t])
 *   completion_lens[s] = sum_t shifted[t]
 * all fp64, each summed in a fixed order (the reference's index_add_ has
 * none).  An empty sequence gives zeros.
 */
int aa_dpo_seq_sums(const float* logp, const float* ref_logp,
                    const uint8_t* loss_mask, const int32_t* cu_seqlens,
                    int64_t n_seqs, int64_t T, double* policy_sums,
                    double* ref_sums, double* completion_lens, void* stream);

/*
 * Backward of aa_dpo_seq_sums in logp (what autograd derives for
 * functional.py:671-673): d_logp[t] = (float)(g_policy_sums[s(t)] * scale[0])
 * * shifted[t]; scale (device, one float) may be NULL for 1.  Tokens outside
 * every sequence get 0.
 */
int aa_dpo_seq_sums_bwd(const double* g_policy_sums, const float* scale,
                        const uint8_t* loss_mask, const int32_t* cu_seqlens,
                        int64_t n_seqs, int64_t T, float* d_logp,
                        void* stream);

/*
 * dpo_preference_loss (functional.py:689-703) on logits already cast to
 * float32 (the reference's first step): loss_type 0 ("sigmoid")
 * loss = -logsigmoid(beta * x); 1 ("ipo") loss = (x - 1 / (2 beta))^2.
 * dloss = d loss / d x, may be NULL.
 */
int aa_dpo_preference_loss(const float* logits, int64_t n, double beta,
                           int loss_type, float* loss, float* dloss,
                           void* stream);

/*
 * The rest of compute_dpo_loss (areal/trainer/dpo/dpo_engine.py:147-213) from
 * the per-sequence sums, for n_pairs = n_seqs / 2 pairs: a pair is valid when
 * both of its sequences are non-empty (_dpo_valid_pairs, :22-24); its logit is
 * (policy_c - policy_r) - (ref_c - ref_r) for loss_type 0 and the difference
 * of the per-token averages (policy - ref) / max(len, 1) for loss_type 1, in
 * fp64, then the loss above in float32.  loss_mean[0] = mean over the valid
 * pairs (0 when there are none), n_valid[0] their number; per pair
 * pair_loss, chosen_reward = beta * (policy_c - ref_c), rejected_reward, valid
 * (zeros for an invalid pair); g_policy_sums [2 * n_pairs] =
 * d loss_mean / d policy_sums.
 */
int aa_dpo_pair_loss(const double* policy_sums, const double* ref_sums,
                     const double* completion_lens, const int32_t* cu_seqlens,
                     int64_t n_pairs, double beta, int loss_type,
                     float* loss_mean, int32_t* n_valid, float* pair_loss,
                     float* chosen_reward, float* rejected_reward,
                     uint8_t* valid, double* g_policy_sums, void* stream);

/*
 * Rows of the table aa_logging_stats writes; each row is {sum, min, max,
 * count} over the selected tokens (min = +inf, max = -inf, count = 0 when
 * nothing is selected or the quantity was not asked for).
 *   0      prox_logp_gt
 *   1..3   kl_div_direct = -(logp - old), kl_div_taylor = (logp - old)^2 / 2,
 *          kl_div_dual = exp(logp - old) - 1 - (logp - old)
 *   4 + 10 m + j, method m = 0 loglinear, 1 linear, 2 rollout:
 *          j = 0 approx_logp, 1 behave_imp_weight = exp(approx - old),
 *          2 importance_weight = exp(logp - approx), 3 abs_error,
 *          4 rel_error, 5 squared_error (of approx against prox_logp_gt),
 *          6 behave_imp_weight_abs_error, 7 behave_imp_weight_rel_error,
 *          8 importance_weight_abs_error, 9 importance_weight_rel_error
 *   34, 35 sample staleness (current_version - 1) - version and
 *          current_version - version over the selected tokens with
 *          version >= 0
 */
#define AA_LOGSTAT_SLOTS 36

/* Bytes of 256-byte aligned scratch aa_logging_stats needs for n tokens. */
int64_t aa_logging_stats_scratch_bytes(int64_t n);

/*
 * The per-token quantities _log_proximal_approximation_stats and
 * _log_version_staleness_stats (areal/trainer/ppo/actor.py:982-1110, helpers
 * :859-979) hand to the statistics tracker, reduced under mask in one pass.
 * prox_logp_gt may be NULL (row 0 and the error rows stay empty; with_errors
 * must be 0); versions (int32, negative for prompt tokens) may be NULL when
 * methods == 0 (then rows 1..3 and 34, 35 stay empty, as the reference
 * returns before logging them).  methods: bit m selects method m of
 * aa_prox_logp_approx.  An error is |gt - a|, |(gt - a) / (|gt| + 1e-8)|,
 * (gt - a)^2.  out [AA_LOGSTAT_SLOTS, 4] float32.
 */
int aa_logging_stats(const float* old_logp, const float* logp,
                     const float* prox_logp_gt, const int32_t* versions,
                     const uint8_t* mask, int64_t n, int current_version,
                     int methods, int with_errors, float* out, void* scratch,
                     int64_t scratch_bytes, void* stream);

/*
 * compute_rw_loss (areal/trainer/rw/rw_engine.py:115-146) over a packed batch
 * of interleaved (chosen, rejected) sequences: the score of a sequence is
 * scores[cu_seqlens[s + 1] - 1]; a pair is valid when both sequences are
 * non-empty (:20-22).  Per pair: pair_loss = -logsigmoid(pos - neg),
 * pos_score, neg_score, valid (zeros for an invalid pair); loss_mean[0] = mean
 * over the valid pairs (0 when there are none), n_valid[0] their number;
 * g_scores [T] = d loss_mean / d scores (nullable).
 */
int aa_rw_pair_loss(const float* scores, int64_t T, const int32_t* cu_seqlens,
                    int64_t n_pairs, float* loss_mean, int32_t* n_valid,
                    float* pair_loss, float* pos_score, float* neg_score,
                    uint8_t* valid, float* g_scores, void* stream);

/* Bytes of 256-byte aligned workspace aa_m2po_mask needs for n tokens. */
int64_t aa_m2po_workspace_bytes(int64_t n);

/*
 * _apply_m2po_masking (areal/trainer/ppo/actor.py:769-850): among the tokens
 * with mask_in != 0, clear those with the largest (old_logp - prox_logp)^2
 * until the mean of the rest is below m2_threshold (at least one token is
 * kept).  mask_out [n] bytes; info[0] = selected tokens, info[1] = tokens
 * cleared.  Equal values are cleared in index order.
 */
int aa_m2po_mask(const float* old_logp, const float* prox_logp,
                 const uint8_t* mask_in, int64_t n, float m2_threshold,
                 uint8_t* mask_out, int32_t* info, void* workspace,
                 int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ */
/* Advantage pipeline (rows are sequences of a padded [bs, L] batch)      */
/* ------------------------------------------------------------------ */

/*
 * GAE reverse scan of PPOActor._compute_advantages
 * (areal/trainer/ppo/actor.py:209-236), which the reference runs as a Python
 * loop over max_seqlen.  For t = L-2 .. 0, with nv = values[:, L-1] *
 * seq_no_eos and lg = 0 to start:
 *   delta = rewards[t] + discount * nv - values[t]
 *   new   = delta + discount * gae_lambda * lg
 *   nv    = nv * (1 - m[t]) + values[t] * m[t]
 *   lg    = lg * (1 - m[t]) + new * m[t];   advantages[t] = lg
 * advantages[:, L-1] = 0; returns = advantages + values (nullable).
 * rewards, loss_mask [bs, L] float32 contiguous; values nullable (zeros);
 * seq_no_eos [bs] bytes, nullable (zeros).  One wave per row: the
 * recurrence is an affine map per token, composed by a wave-level scan.
 */
int aa_gae(const float* rewards, const float* values, const float* loss_mask,
           const uint8_t* seq_no_eos, int64_t bs, int64_t L, float discount,
           float gae_lambda, float* advantages, float* returns, void* stream);

/*
 * KL-regularised token rewards of PPOActor._compute_advantages
 * (areal/trainer/ppo/actor.py:182-207) for a padded [bs, L] batch:
 *   kl_rewards = -kl_ctl * KL(old_logp * m, ref_logp * m), estimator 0 = k1,
 *                1 = k2, 2 = k3, clamped to [-10, 10] (areal/utils/data.py:1620-1656)
 *   rewards    = kl_rewards, with position seqlens[b] - 1 cleared and
 *                reward_score[b] added at position max(seqlens[b] - 2, 0)
 *                (not added when mask_no_eos_with_zero and seqlens[b] == L).
 * ref_logp may be NULL (zeros).  loss_mask is the float mask already rolled.
 */
int aa_kl_rewards(const float* old_logp, const float* ref_logp,
                  const float* loss_mask, const int64_t* seqlens,
                  const float* reward_score, int64_t bs, int64_t L,
                  float kl_ctl, int estimator, int mask_no_eos_with_zero,
                  float* rewards, float* kl_rewards, void* stream);

/* Normalization (areal/utils/data.py:1378-1596); levels: 0 none, 1 batch,
 * 2 group; mirrors NormConfig (areal/api/cli_args.py:42-95). */
typedef struct {
  int32_t mean_level;
  int32_t mean_leave1out;
  int32_t std_level;
  int32_t std_unbiased;
  float eps;
  int64_t group_size; /* rows per group, used when a level is 2 */
} aa_norm_params;

/* Bytes of scratch aa_normalize needs (32-byte aligned device memory). */
int64_t aa_normalize_scratch_bytes(int64_t bs, int64_t inner,
                                   int64_t group_size);

/*
 * out = Normalization(params)(x, loss_mask) for x [bs, inner] float32
 * contiguous and an optional float32 mask of the same shape: centring by the
 * batch / group mean (optionally leave-one-out), masking, division by the
 * batch / group standard deviation (+ eps).  Sums are accumulated in float64
 * in a fixed order; group-level means and deviations are rounded to float32
 * where the reference stores them in float32 tensors.  Rows past the last
 * full group keep mean = std = 0, and an all-zero mask returns x, both as in
 * the reference.
 */
int aa_normalize(const float* x, const float* loss_mask, int64_t bs,
                 int64_t inner, const aa_norm_params* params, float* out,
                 void* scratch, int64_t scratch_bytes, void* stream);

/*
 * Masked moments of up to 16 per-token float32 tensors under one byte mask,
 * the reductions the statistics logger performs one tensor at a time
 * (areal/utils/stats_tracker.py:227-285): out[k] = {sum, min, max, count}
 * over mask != 0 (min = +inf, max = -inf when the mask is empty).
 * values is a HOST array of n_tensors device pointers.
 */
int aa_masked_moments(const float* const* values, int n_tensors,
                      const uint8_t* mask, int64_t n, float* out, void* stream);

/* ------------------------------------------------------------------ */
/* Fused lm_head path (no counterpart in the reference: its equivalent is  */
/* logits = hidden @ weight.T followed by the logits path above)           */
/* ------------------------------------------------------------------ */

/* Bytes of workspace aa_lmhead_bwd / aa_lmhead_ppo_fused need for these sizes.
 * With C = min(T, aa_lmhead_chunk_tokens()): 2 * C * V (the bf16 d(logits)
 * rows of one token chunk; their pitch is V rounded up to 8), 32 * (V / 256) *
 * C (softmax partials and smallest logit per 128 vocabulary rows and token), 2 * C * H (the hidden rows of the tokens with a
 * gradient, closed up), 16 * C * H (four fp32 planes of d_hidden rows: the
 * product that forms them has few tiles and is cut along the vocabulary into
 * up to four parts when that fills the chip better), plus 4 * H * V (an fp32
 * accumulator for a bf16 d_weight) when there is more than one chunk.  No
 * transposed copy of anything is made.  Returns -1 for sizes the path does
 * not take. */
int64_t aa_lmhead_workspace_bytes(int64_t T, int64_t H, int64_t V);

/* Bytes of workspace aa_lmhead_fwd alone needs: the softmax partials only,
 * about 24 * (V / 256) * min(T, aa_lmhead_chunk_tokens()) bytes (0.23 GB at
 * T = 16384, V = 151936). */
int64_t aa_lmhead_fwd_workspace_bytes(int64_t T, int64_t H, int64_t V);

/* The same when aa_lmhead_fwd is also asked for vocab_max / vocab_min: one
 * more plane, the smallest logit per 128 vocabulary rows and token (a third
 * more). */
int64_t aa_lmhead_fwd_stats_workspace_bytes(int64_t T, int64_t H, int64_t V);

/* Tokens per chunk of the lm_head entry points (16384). */
int64_t aa_lmhead_chunk_tokens(void);

/*
 * Per-device set-up of the lm_head entry points (the tile kernels are allowed
 * their 160 KiB of LDS with hipFuncSetAttribute, which is not a stream
 * operation).  Every aa_lmhead_* entry point does it by itself on its first
 * call on a device; call this once per device, with that device current,
 * before capturing any of them into a HIP graph, so that no such call falls
 * inside the capture.  No counterpart in the reference.
 */
int aa_lmhead_prepare(void);

/*
 * logp / entropy of softmax(hidden @ weight.T / temperature) without writing
 * the logits anywhere: 256 x 256 tiles of them are formed in the accumulator
 * registers of this library's bf16 MFMA tile GEMM (fp32 accumulation, no
 * rounding to bf16 in between), each tile is reduced to softmax partials per
 * token in the GEMM's epilogue, and a small kernel merges the partials.
 * hidden [T, H] bf16 row-major, weight [V, H] bf16 row-major; H a multiple of
 * 8, any V (both below 2^22), as the reference's lm_head ->
 * _gather_logprobs_entropy (areal/utils/functional/vocab_parallel.py:23-29)
 * takes any vocabulary.  entropy, row_lse, row_ez may be NULL; row_lse / row_ez
 * as in aa_logits_fwd (needed by aa_lmhead_bwd).
 * vocab_max / vocab_min [T] (both or neither): largest and smallest logit of
 * every row, what FSDPEngine._get_vocab_min_max_logits reads from materialised
 * logits (areal/engine/fsdp_engine.py:1893-1906), here from the fp32 sums of
 * the tiles (the smallest exactly; the largest through the softmax exponent,
 * i.e. to one rounding).
 * workspace: aa_lmhead_fwd_workspace_bytes(T, H, V) bytes, or
 * aa_lmhead_fwd_stats_workspace_bytes(T, H, V) with the extrema.
 */
int aa_lmhead_fwd(const void* hidden, const void* weight, int64_t T, int64_t H,
                  int64_t V, const int64_t* labels, float inv_temperature,
                  float* logp, float* entropy, float* row_lse, float* row_ez,
                  float* vocab_max, float* vocab_min, void* workspace,
                  int64_t workspace_bytes, void* stream);

/*
 * aa_lmhead_fwd for callers that cannot allocate device memory or bring a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  No counterpart in the reference.  Same arguments and
 * results as aa_lmhead_fwd without the workspace and the vocabulary extrema: the softmax partials live in
 * a device array of the library itself, aa_lmhead_fwd_static_scratch_bytes()
 * = 32 MiB on every GPU the library has been used on, held until the process
 * ends.  Tokens go through in passes of as many as fit that array (a multiple
 * of 256; 2304 per pass at V = 151936); a vocabulary above
 * aa_lmhead_fwd_static_max_vocab() (1 398 016), for which not even 256 tokens
 * fit, is refused with AA_ERR_UNSUPPORTED.  The call allocates and frees
 * nothing.  All calls on one GPU share the array: calls that overlap on one GPU
 * (two streams, two host threads) race and must be serialised by the caller;
 * nothing in the array needs clearing between calls.  The first call on a
 * device also does that device's set-up (aa_lmhead_prepare and the address of
 * the array, neither a stream operation): make one eager call, or call
 * aa_lmhead_prepare and then this once, before capturing it into a graph.
 */
int aa_lmhead_fwd_static(const void* hidden, const void* weight, int64_t T,
                         int64_t H, int64_t V, const int64_t* labels,
                         float inv_temperature, float* logp, float* entropy,
                         float* row_lse, float* row_ez, void* stream);
int64_t aa_lmhead_fwd_static_scratch_bytes(void);
int64_t aa_lmhead_fwd_static_max_vocab(void);

/*
 * Backward of aa_lmhead_fwd: d_hidden [T, H] bf16 and d_weight [V, H]
 * (overwritten), given g_logp and optional g_entropy.  d_weight_dtype is
 * AA_F32 or AA_BF16; either way the sum over tokens is accumulated in fp32
 * (bf16: rounded once at the end).
 * Per chunk of tokens: the logits tiles are formed again and turned into
 * bf16 d(logits) rows in the GEMM's epilogue (a panel [rows, V] in the
 * workspace), which two more tile GEMMs contract with the weight and with the
 * hidden states (6 T V H flops for the 4 T V H of the backward).
 * row_has_gradient [T] (device, one byte per token) with kept_per_chunk (HOST,
 * its non-zero count per chunk of aa_lmhead_chunk_tokens() tokens), both or
 * neither: rows whose byte is zero must have g_logp == 0 and g_entropy == 0;
 * they are left out of all three GEMMs, and a chunk without any other row is
 * skipped altogether.  An entry may be AA_LMHEAD_COUNT_ON_DEVICE.
 * workspace: aa_lmhead_workspace_bytes(T, H, V) bytes.
 */
int aa_lmhead_bwd(const void* hidden, const void* weight, int64_t T, int64_t H,
                  int64_t V, const int64_t* labels, float inv_temperature,
                  const float* row_lse, const float* row_ez,
                  const float* g_logp, const float* g_entropy,
                  const uint8_t* row_has_gradient,
                  const int64_t* kept_per_chunk, void* d_hidden,
                  void* d_weight, int d_weight_dtype, void* workspace,
                  int64_t workspace_bytes, void* stream);

/*
 * The stand-alone op with a backward of two plain GEMMs (no counterpart in the
 * reference, whose autograd keeps the [T, V] logits): aa_lmhead_fwd_carry is
 * aa_lmhead_fwd that also writes, for the tokens that may get a gradient, the
 * bf16 rows p_v / p_label into `panel` (see AA_LMHEAD_CARRY below), and
 * aa_lmhead_bwd_carry turns them into d_hidden and d_weight once g_logp is
 * known: one factor per row, applied inside the two GEMMs; no second logits
 * GEMM.  For losses that need the log-probs of the whole batch before any
 * gradient exists (sequence-level importance ratios, areal/utils/functional/
 * functional.py:56-149; SAPO, :562-638), at the price of keeping the panel
 * between the two calls: panel_rows x aa_lmhead_panel_pitch(V) bf16, with
 * panel_rows >= the sum of kept_per_chunk (or T when that is NULL); the rows of
 * chunk c start after those of the chunks before it.
 * row_has_gradient [T] (device) with kept_per_chunk (HOST), both or neither,
 * as in aa_lmhead_bwd: tokens whose byte is zero get no panel row and no
 * gradient, whatever g_logp holds for them; the same two arrays must be passed
 * to both calls.  An entry of kept_per_chunk may be AA_LMHEAD_COUNT_ON_DEVICE
 * (below): that chunk counts as all of its tokens in panel_rows and in where
 * the next chunk's rows start, and its kernels stop at the rows in use.  An
 * entropy gradient cannot be carried: use aa_lmhead_bwd
 * (row_lse / row_ez of this forward serve it) when there is one.  A chunk with
 * a row that does not fit the stored form is redone from the logits tiles,
 * decided on the device.  logp / row_lse: outputs of the forward, inputs of the
 * backward.  workspace: aa_lmhead_carry_workspace_bytes(T, H, V) bytes for
 * either call (the workspace of aa_lmhead_bwd without its panel).
 */
int64_t aa_lmhead_carry_workspace_bytes(int64_t T, int64_t H, int64_t V);
int64_t aa_lmhead_panel_pitch(int64_t V);
int aa_lmhead_fwd_carry(const void* hidden, const void* weight, int64_t T,
                        int64_t H, int64_t V, const int64_t* labels,
                        float inv_temperature,
                        const uint8_t* row_has_gradient,
                        const int64_t* kept_per_chunk, float* logp,
                        float* entropy, float* row_lse, float* row_ez,
                        float* vocab_max, float* vocab_min, void* panel,
                        int64_t panel_rows, void* workspace,
                        int64_t workspace_bytes, void* stream);
int aa_lmhead_bwd_carry(const void* hidden, const void* weight, int64_t T,
                        int64_t H, int64_t V, const int64_t* labels,
                        float inv_temperature, const float* logp,
                        const float* row_lse, const float* g_logp,
                        const uint8_t* row_has_gradient,
                        const int64_t* kept_per_chunk, void* panel,
                        int64_t panel_rows, void* d_hidden, void* d_weight,
                        int d_weight_dtype, void* workspace,
                        int64_t workspace_bytes, void* stream);

/* A kept_per_chunk entry that leaves the count to the device (aa_lmhead_bwd,
 * aa_lmhead_ppo_fused, aa_lmhead_fwd_carry / aa_lmhead_bwd_carry): the kernels of that chunk are launched for every token
 * that could have a row and stop at the rows in use, which the device counts
 * itself, so the host needs no copy of the mask and does not wait for the
 * device.  The tiles over the rows in use are numbered, and the d_hidden
 * product is cut along the vocabulary or not, exactly as with that count given
 * by the host: the results are the same bits, and the workgroups that find
 * nothing to do return at once (no measurable cost). */
#define AA_LMHEAD_COUNT_ON_DEVICE (-1)

/* How aa_lmhead_ppo_fused fills the d(logits) rows that its backward GEMMs
 * contract. */
typedef enum {
  /* the logits tiles of the tokens with gradient are formed a second time,
   * once the loss is known (2 T_grad V H extra flops; the forward half writes
   * nothing of size T x V) */
  AA_LMHEAD_RECOMPUTE = 0,
  /* the forward tiles also write p_v / p_label (the label logit is known
   * before they run) as bf16 into the rows of the tokens with gradient; once
   * the loss is known, d(logits) of a row is that row times one factor per
   * token, which the two gradient GEMMs apply themselves (no second logits
   * GEMM, no pass over the rows).  A chunk with a token whose label has a
   * log-prob below -80, or whose factor is below 2^-100 in magnitude, does
   * not fit the stored range and is redone as in AA_LMHEAD_RECOMPUTE, decided
   * on the device (same results, slower). */
  AA_LMHEAD_CARRY = 1
} aa_lmhead_backward_mode;

/*
 * Whole training step of the lm_head + PPO actor loss for one micro-batch,
 * token-level importance sampling: what the reference runs as lm_head matmul
 * -> gather_logprobs_entropy (vocab_parallel.py:434-469) ->
 * ppo_actor_loss_fn (functional.py:429-559) -> autograd back to the hidden
 * states and the lm_head weight.  Tokens are processed in chunks of at most
 * aa_lmhead_chunk_tokens().  Per chunk: the forward tiles of aa_lmhead_fwd; one kernel that
 * merges the softmax partials into log-prob and entropy and evaluates the
 * per-token loss and its derivative; the bf16 d(logits) rows of the tokens
 * with gradient (backward_mode says how they are obtained); and the two tile
 * GEMMs that contract those rows with the weight and the hidden states.  The
 * logits themselves are never written to memory.
 *
 * Per-token arguments, params, n_valid, grad_scale: as in
 * aa_logits_ppo_fused.  d_hidden [T, H] bf16 and d_weight [V, H] (AA_F32 or
 * AA_BF16, fp32 accumulation either way, as in aa_lmhead_bwd) are
 * overwritten.  workspace: aa_lmhead_workspace_bytes(T, H, V) bytes.
 *
 * kept_per_chunk (HOST memory, nullable): a token whose mask_eff is zero has
 * a zero gradient row, so it adds nothing to d_weight and its d_hidden row is
 * zero.  Given, for every chunk of aa_lmhead_chunk_tokens() tokens, the number
 * of non-zero mask_eff bytes among the chunk's first min(T_active - t0, chunk)
 * tokens, only those tokens get a d(logits) row and go through the backward
 * GEMMs (the reference's autograd multiplies the zero rows through).  The
 * counts size the GEMMs, which is why they come from the host; tokens beyond a
 * count that is too small are treated as masked, and the surplus rows of a
 * count that is too large are cleared on the device and add nothing (slower,
 * same results).  An entry may be AA_LMHEAD_COUNT_ON_DEVICE: no host count
 * is needed then.  NULL: every token has a row.
 * vocab_max / vocab_min [T] (nullable, both or neither): as in aa_lmhead_fwd.
 */
int aa_lmhead_ppo_fused(const void* hidden, const void* weight, int64_t T,
                        int64_t H, int64_t V, const int64_t* labels,
                        float inv_temperature, int64_t T_active,
                        const float* prox_logp, const float* adv,
                        const uint8_t* mask_eff, const float* behave_w,
                        const aa_ppo_params* params, const int32_t* n_valid,
                        const float* grad_scale, const int64_t* kept_per_chunk,
                        int backward_mode, float* logp, float* entropy,
                        float* stat_loss, float* ratio, uint8_t* flags,
                        float* vocab_max, float* vocab_min, void* d_hidden,
                        void* d_weight, int d_weight_dtype, void* workspace,
                        int64_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ */
/* Packing                                                                 */
/* ------------------------------------------------------------------ */

/*
 * Segmented row copy, the data movement of pack_tensor_dict,
 * pad_packed_tensor_dict and unpad_logits (areal/utils/data.py:492-541,
 * 818-978, 1046-1074), which the reference does with one slice assignment
 * per sequence.  Rows (tokens) have row_bytes bytes.  seg_cu [B+1] int32:
 * seg_cu[i] = rows in segments before i (seg_cu[B] = total_rows); row o of
 * segment i is copied from src row src_starts[i] + o to dst row
 * dst_starts[i] + o.  All index arrays live on the device.  Rows of dst that
 * no segment covers are left untouched.
 */
int aa_segment_copy(const void* src, void* dst, int64_t row_bytes,
                    const int64_t* src_starts, const int64_t* dst_starts,
                    const int32_t* seg_cu, int64_t B, int64_t total_rows,
                    void* stream);

/* ------------------------------------------------------------------ */
/* Measurement helper                                                  */
/* ------------------------------------------------------------------ */

/* dst[0..nbytes) = src[0..nbytes), 16-byte aligned, nbytes % 16 == 0: the
 * plain copy the HBM counters of the other kernels are calibrated against. */
int aa_copy_bytes(const void* src, void* dst, int64_t nbytes, void* stream);

/* A loop of nothing but bf16 MFMAs on operands that stay in registers (no LDS,
 * no memory traffic): what the matrix cores of this chip sustain at its power
 * limit, the measured ceiling beside the MFMA-bound kernels.  form 0:
 * v_mfma_f32_32x32x16_bf16, 16 per wave and iteration; form 1:
 * v_mfma_f32_16x16x32_bf16, 64 per wave and iteration; 4 waves per workgroup,
 * so an iteration is 2 097 152 (form 0) or 4 194 304 (form 1) flops per
 * workgroup.  random_operands: random signs and mantissas (as activations
 * are) or zeros.  out [workgroups * 256] receives a checksum per lane.  No
 * counterpart in the reference; not on any product path. */
int aa_mfma_only_loop(int form, int random_operands, int workgroups, int iters,
                      float* out, void* stream);

/* Plain streams over `bytes` bytes (a multiple of 16, 16-byte aligned), the
 * measured ceilings beside the HBM-bound kernels: kind 0 reads src (nothing
 * is written; dst may be NULL), kind 1 writes dst (src may be NULL), kind 2
 * copies src to dst.  nt_policy != 0 selects the streaming (`nt`) cache
 * policy for the loads and stores.  `workgroups` workgroups of 256 threads
 * deal 32 KB pieces among themselves.  No counterpart in the reference; not on
 * any product path. */
int aa_hbm_stream_probe(int kind, int nt_policy, const void* src, void* dst,
                        int64_t bytes, int workgroups, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AREAL_AMD_H */
