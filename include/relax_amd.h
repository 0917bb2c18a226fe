/*
 * relax_amd -- C ABI of the MI355X (gfx950) kernels for Relax's per-token
 * log-prob / entropy / policy-loss / advantage path.
 *
 * The reference (redai-infra/Relax) has no FFI for this path: it is pure
 * PyTorch.  Each entry point below therefore cites the reference Python
 * function whose arithmetic it replaces (paths relative to the reference
 * checkout).  Conventions:
 *   - all pointers are DEVICE pointers unless stated otherwise; the caller
 *     owns every buffer; outputs are caller-allocated; inputs are never
 *     written;
 *   - no entry point allocates, frees or synchronises; work is enqueued on
 *     `stream` (a hipStream_t passed as void*; NULL = the default stream);
 *   - return value 0 = success, negative = error; the message is available
 *     from relax_amd_last_error() on the calling thread;
 *   - `dtype` is one of the RELAX_AMD_* element codes; fp32 is used for all
 *     per-token side vectors;
 *   - kernels are deterministic (no floating-point atomics): the same inputs
 *     give bit-identical outputs run to run.
 */
#ifndef RELAX_AMD_H
#define RELAX_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* 2: relax_amd_policy_loss_args starts with its own size and carries the top-K distillation block and
 *    read_masked_rows; relax_amd_set_kernel_choice replaces the environment switch; relax_amd_transpose_16bit,
 *    relax_amd_diag_mfma_loop and relax_amd_diag_stream are gone.  A client built against version 1 must be rebuilt. */
#define RELAX_AMD_ABI_VERSION 2

enum { RELAX_AMD_F32 = 0, RELAX_AMD_BF16 = 1, RELAX_AMD_F16 = 2, RELAX_AMD_F64 = 3 };

enum { RELAX_AMD_OK = 0, RELAX_AMD_EINVAL = -1, RELAX_AMD_ELAUNCH = -2, RELAX_AMD_EUNSUPPORTED = -3 };

/* policy-loss flavours (relax/backends/megatron/loss.py:976-1000) */
enum { RELAX_AMD_LOSS_PPO = 0, RELAX_AMD_LOSS_GSPO = 1, RELAX_AMD_LOSS_CISPO = 2, RELAX_AMD_LOSS_RLOO = 3, RELAX_AMD_LOSS_SAPO = 4 };
/* KL estimators (relax/utils/training/ppo_utils.py:100-139) */
enum { RELAX_AMD_KL_NONE = 0, RELAX_AMD_KL_K1 = 1, RELAX_AMD_KL_K2 = 2, RELAX_AMD_KL_K3 = 3, RELAX_AMD_KL_LOW_VAR = 4 };
/* group reward normalisation (relax/utils/utils.py:199-238) */
enum { RELAX_AMD_GROUP_CENTER = 0, RELAX_AMD_GROUP_CENTER_STD = 1, RELAX_AMD_GROUP_RLOO = 2 };
/* top-K distillation signal: the JSD family (jsd_alpha 0 = reverse KL, 1 = forward KL) or the element-wise k3 sum */
enum { RELAX_AMD_OPD_JSD = 0, RELAX_AMD_OPD_LOW_VAR = 1 };
/* opd_norm_mode: append the tail bin log(1 - sum p), renormalise over the K entries, or use them as they are */
enum { RELAX_AMD_OPD_NORM_TAIL = 0, RELAX_AMD_OPD_NORM_NORM = 1, RELAX_AMD_OPD_NORM_TRUNC = 2 };

/* slots of the metrics vector written by relax_amd_policy_loss */
enum {
  RELAX_AMD_M_LOSS = 0,
  RELAX_AMD_M_PG_LOSS = 1,
  RELAX_AMD_M_ENTROPY = 2,
  RELAX_AMD_M_CLIPFRAC = 3,
  RELAX_AMD_M_PPO_KL = 4,
  RELAX_AMD_M_KL_LOSS = 5,
  RELAX_AMD_M_LOGPROB_ABS_DIFF = 6,
  RELAX_AMD_M_PROB_ABS_DIFF = 7,
  RELAX_AMD_M_OIS = 8,
  RELAX_AMD_M_TIS = 9,
  RELAX_AMD_M_TIS_CLIPFRAC = 10,
  RELAX_AMD_M_TIS_ABS = 11,
  RELAX_AMD_M_MISMATCH_KL = 12,
  RELAX_AMD_M_MISMATCH_K3 = 13,
  RELAX_AMD_M_OPSM_CLIPFRAC = 14,
  RELAX_AMD_M_MASK_SUM = 15,
  RELAX_AMD_NUM_METRICS = 16
};

int relax_amd_version(void);
/* Message of the last failing call on this thread ("" if none). Host pointer, valid until the next call. */
const char* relax_amd_last_error(void);

/* which of their bit-identical kernels the fused entry points launch (see relax_amd_set_kernel_choice) */
enum { RELAX_AMD_KERNEL_AUTO = 0, RELAX_AMD_KERNEL_TWO_WALK = 1, RELAX_AMD_KERNEL_RESIDENT = 2 };
/*
 * relax_amd_actor_step_fused, relax_amd_logprob_entropy_bwd and relax_amd_reverse_kl_step_fused each hold a
 * persistent register-resident kernel for the row lengths it is built for and a two-walk (row-per-workgroup) kernel
 * for every row length; each also holds a kernel of one-shot workgroups in address order (the actor step and the
 * reverse-KL step: eight workgroups share a row and exchange their partial softmax sums through a ring in device
 * memory; the backward: one workgroup per 4 KB of a row).  All give the same bits.  AUTO (the default) takes the one-shot form
 * where it exists, else the resident one, else the two-walk kernel.  TWO_WALK keeps every row on the two-walk
 * kernel; RESIDENT takes the persistent kernel and makes those entry points fail with RELAX_AMD_EUNSUPPORTED where
 * none is built, so that a comparison of kernels cannot pass on one kernel compared with itself.
 * Process-wide, read atomically at each launch; returns the previous choice, or RELAX_AMD_EINVAL.  No counterpart
 * in the reference: it exists for tests and measurements.
 *
 * The one-shot kernels of the actor step and of the reverse-KL step each keep their exchange ring (1.5 MB, plus 8 MB
 * for the logits gathered at a row's top-K ids / 2.5 MB) in static arrays of the library, one copy per GPU and process.  Launches of the same entry point that overlap on
 * one GPU (two streams of one process) must not both take that kernel: they could overwrite each other's slots, which
 * the kernel notices (bounded waits) and reports as NaN log-probs (NaN KL) rather than wrong numbers.  Launches in stream order, captured graphs and their replays
 * are fine (the tags that tell one launch's partial sums from another's come from a counter in device memory that a
 * small kernel in front of each launch advances); the first call on a GPU looks the ring's address up
 * (hipGetSymbolAddress), so make one call outside a capture first.
 */
int relax_amd_set_kernel_choice(int choice);
/*
 * Which kernel family the last launching call on this thread ended with ("" before any): "actor_step_split",
 * "actor_step_resident", "actor_step_resident_wide" or "actor_step_fused" (the two-walk kernel) after
 * relax_amd_actor_step_fused; "reverse_kl_split", "reverse_kl_resident" or "reverse_kl_step_fused" after
 * relax_amd_reverse_kl_step_fused; "logprob_entropy_bwd_chunk", "logprob_entropy_bwd_resident" or
 * "logprob_entropy_bwd" after relax_amd_logprob_entropy_bwd; the entry point's own name elsewhere.  Host pointer to a
 * constant string.  No counterpart in the reference: it lets a caller (and this library's tests) see that a row shape
 * took the kernel built for it rather than the two-walk kernel, which serves every shape with the same results.
 */
const char* relax_amd_last_kernel(void);

/*
 * For tests of the failure handling of the one-shot actor and reverse-KL steps: max_polls bounds how often a workgroup looks for its
 * neighbours' partial sums before it gives up (0 = the default), wait_tag_offset is added to the tag it looks
 * for (0 = none; with 1 no wait can succeed; the default bound is 2^17 looks, and the first give-up of a launch ends
 * the launch's other waits at their next check of a flag).  A launch made with (a few, 1) therefore exercises the give-up path on
 * every row without any workgroup hanging: log-probs and log-sum-exps of the scored tokens (the reverse-KL step: KL
 * and both log-sum-exps of every token) come back NaN.
 * Process-wide, read at each launch.  No counterpart in the reference.
 */
int relax_amd_set_exchange_wait(int max_polls, int wait_tag_offset);

/*
 * Target-token log-prob and full-vocab entropy of each row, one streaming
 * read of the row.  Replaces _VocabParallelLogProbEntropy.forward
 * (relax/utils/training/ppo_utils.py:481-589, single vocab shard) together
 * with the per-sample temperature division of get_responses
 * (relax/backends/megatron/loss.py:184-189).
 *   logits      [*, vocab] elements of `dtype`, row r at logits + row*row_stride
 *   row_ids     [n_tokens] int32 logits-row of each token, or NULL (token i = row i)
 *   targets     [n_tokens] int64 target id of each token (ids outside [0,vocab) give NaN)
 *   log_prob    [n_tokens] out: (x[target] - logsumexp(x)) with x = logits * inv_temperature
 *   entropy     [n_tokens] out or NULL: logsumexp(x) - sum_v softmax(x)*x
 *   lse, spx    [n_tokens] out or NULL: logsumexp(x) and sum_v softmax(x)*x, consumed by the backward
 */
int relax_amd_logprob_entropy_fwd(const void* logits, int dtype, int64_t n_tokens, int64_t vocab, int64_t row_stride,
                                  const int32_t* row_ids, const int64_t* targets, float inv_temperature,
                                  float* log_prob, float* entropy, float* lse, float* spx, void* stream);

/*
 * dlogits of the forward above, one read of the row and one write.  Replaces
 * _VocabParallelLogProbEntropy.backward (ppo_utils.py:591-629):
 *   dlogits[row] = inv_T * ( g_lp*(onehot(target) - p) + g_ent * p * (spx - x) ),  p = exp(x - lse)
 * Every one of the n_rows logits rows is written exactly once: rows whose
 * token_of_row is negative (prompt / padding positions) and rows whose
 * incoming gradients are both zero are filled with zeros without reading.
 *   token_of_row [n_rows] int32 token index of each logits row, -1 = no token; NULL = identity
 *   g_lp, g_ent  [n_tokens] incoming gradients of log_prob / entropy (g_ent may be NULL)
 *   grad_scale   host scalar multiplied into both incoming gradients
 *   grad_scale_dev optional device scalar (fp32) multiplied in as well, so an upstream autograd scalar needs no
 *                host read-back; NULL = 1
 *   dlogits      [n_rows, vocab] out, elements of `dtype`, row stride d_row_stride
 */
int relax_amd_logprob_entropy_bwd(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                  const int32_t* token_of_row, const int64_t* targets, const float* lse,
                                  const float* spx, const float* g_lp, const float* g_ent, float grad_scale,
                                  const float* grad_scale_dev, float inv_temperature, void* dlogits,
                                  int64_t d_row_stride, void* stream);

/*
 * Row maps of the packed ("thd") response layout.  Replaces the per-sample
 * index arithmetic of get_responses (loss.py:103-125, cp_size == 1) and
 * compute_sft_response_chunk (relax/utils/sft_utils.py:23-40).
 *   row_begin  [n_samples] int64 first logits row that scores sample i's response
 *   cu_resp    [n_samples+1] int64 exclusive prefix sum of response lengths
 *   row_ids    [n_tokens] out int32
 *   sample_ids [n_tokens] out int32 (may be NULL)
 *   token_of_row [n_rows] out int32 or NULL: inverse map, -1 where no response token
 */
int relax_amd_build_row_maps(const int64_t* row_begin, const int64_t* cu_resp, int64_t n_samples, int64_t n_tokens,
                             int64_t n_rows, int32_t* row_ids, int32_t* sample_ids, int32_t* token_of_row,
                             void* stream);

/*
 * Packed target ids of the response tokens in one launch: the per-sample `tokens[-response_length:]` of get_responses
 * (loss.py:103-125) and the shifted, zero-padded `tokens[1:]` of the SFT layout (relax/utils/sft_utils.py:23-40).
 *   tokens     int64, every sample's token ids back to back
 *   src_begin  [n_samples] int64 position in `tokens` of sample i's first target
 *   src_end    [n_samples] int64 end of sample i's tokens; targets past it read as 0
 *   cu_resp    [n_samples+1] int64 exclusive prefix sum of response lengths
 *   targets    [n_tokens] out int64
 */
int relax_amd_gather_targets(const int64_t* tokens, const int64_t* src_begin, const int64_t* src_end,
                             const int64_t* cu_resp, int64_t n_samples, int64_t* targets, void* stream);

/*
 * Per-token policy loss, KL penalty, masked per-sample aggregation and the
 * gradient coefficients d loss / d log_prob, d loss / d entropy.  Replaces the
 * arithmetic of policy_loss_function (loss.py:961-1134) with
 * compute_policy_loss / compute_gspo_kl / compute_cispo_loss / compute_rloo_loss
 * / compute_sapo_loss / compute_approx_kl / compute_opsm_mask
 * (ppo_utils.py:100-396), vanilla_tis_function (loss.py:741-769) and the
 * reducers of get_sum_of_sample_mean (relax/backends/megatron/cp_utils.py:144-162).
 */
typedef struct relax_amd_policy_loss_args {
  /* sizeof(relax_amd_policy_loss_args) as the caller was compiled; a smaller value than the library's own is
     refused with RELAX_AMD_EINVAL before any field behind it is read */
  uint32_t struct_size;
  uint32_t reserved;             /* 0 */
  /* packed per-token inputs, fp32 [n_tokens]; NULL where marked optional */
  const float* log_prob;
  const float* old_log_prob;     /* NULL: old = current (true on-policy, ratio == 1) */
  const float* ref_log_prob;     /* optional: needed when kl_type != NONE */
  const float* train_log_prob;   /* optional: train-engine log-probs for TIS / mismatch metrics (NULL = current) */
  const float* rollout_log_prob; /* optional */
  const float* advantages;
  const float* loss_mask;        /* mask values as fp32 (multiplied, not tested) */
  const float* pg_loss_mask;     /* optional: numerator mask of the pg-loss reducer (NULL = loss_mask) */
  const float* entropy;          /* optional */
  const int64_t* cu_resp;        /* [n_samples+1] */
  const float* sample_denom;     /* [n_samples] divisor of each sample's masked sum (already clamped), NULL = 1 */
  const float* pg_sample_denom;  /* [n_samples] divisor for pg_loss only, NULL = sample_denom */
  int64_t n_samples;
  int64_t n_tokens;
  int32_t loss_kind;             /* RELAX_AMD_LOSS_* */
  int32_t kl_kind;               /* RELAX_AMD_KL_* */
  int32_t unbiased_kl;           /* multiply KL by exp(lp - old), gradient flows through the ratio */
  int32_t use_opsm;
  int32_t use_tis;               /* apply clamp(exp(train - rollout), tis_lo, tis_hi) to pg_loss */
  int32_t mismatch_metrics;      /* emit OIS/TIS metrics */
  int32_t abs_diff_from_old;     /* 1: |old - rollout| metrics use old_log_prob, 0: train_log_prob, 2: current */
  float eps_clip, eps_clip_high, eps_clip_c; /* eps_clip_c <= 0: no dual clip */
  float entropy_coef, kl_coef;
  float tis_lo, tis_hi, opsm_delta, tau_pos, tau_neg;
  /* outputs */
  float* coef_log_prob;          /* [n_tokens] d loss / d log_prob */
  float* coef_entropy;           /* [n_tokens] d loss / d entropy, may be NULL */
  float* pg_loss_tok;            /* optional per-token outputs [n_tokens] */
  float* clipfrac_tok;
  float* ppo_kl_tok;
  float* kl_tok;
  float* sample_partials;        /* workspace [n_samples * RELAX_AMD_NUM_METRICS] */
  float* metrics;                /* [RELAX_AMD_NUM_METRICS] */
  /* optional input, last so that the fields above keep their offsets: [n_tokens] added to d loss / d log_prob of every
   * token whose masks are not both zero -- the gradient of a caller's loss term that is linear in the log-probs, such
   * as opd_loss_coef * token_mean(log_prob - teacher_log_prob) (relax/utils/opd/opd_utils.py:1368-1455 with the
   * sampled-token reverse_kl signal), so that term's gradient leaves in the same dlogits launch.  NULL = none. */
  const float* extra_coef_log_prob;
  /* optional: the sampled-token distillation signal of compute_policy_opd_loss (opd_utils.py:1368-1455) when it is
   * not linear.  With distill_teacher_log_prob [n_tokens] set, extra_coef_log_prob[t] is the weight of token t's
   * signal in the loss (opd_loss_coef * mask / clamp_min(sum mask, 1)) and the kernel multiplies it by the signal's
   * derivative: both log-probs clamped from below at distill_min_clamp, estimator distill_kl_kind (RELAX_AMD_KL_K1
   * for "reverse_kl", RELAX_AMD_KL_K3 for "low_var_kl"), signal clipped from above at distill_token_clip, times
   * min(exp(log_prob - old_log_prob), distill_is_clip) taken as a constant.  A NaN switches a clamp / clip off. */
  const float* distill_teacher_log_prob;
  int32_t distill_kl_kind;
  float distill_min_clamp, distill_token_clip, distill_is_clip;
  /* optional, relax_amd_actor_step_fused only (relax_amd_policy_loss leaves the signal out: with topk_ids set it
   * treats extra_coef_log_prob as absent and touches none of the topk_* fields): the top-K distillation signal of
   * compute_policy_opd_loss (opd_utils.py:1368-1455 with compute_log_probs_on_topk_token_ids, :1022-1094, and
   * compute_opd_kl_topk, :1190-1228) evaluated next to each row's log-sum-exp, so that its gradient leaves in the
   * step's one dlogits launch.  With topk_ids set, extra_coef_log_prob[t] is the weight of token t's signal in the
   * loss; the kernel gathers the row's logits at topk_ids[t, :], forms the per-token KL, clips it from above at
   * distill_token_clip, multiplies by min(exp(log_prob - old_log_prob), distill_is_clip) taken as a constant (NaN
   * switches either off), writes the un-clipped signal to topk_kl[t] and d loss / d log p[id_k] to topk_grad[t, k],
   * and adds the sum of the latter to the multiple of the row's softmax it subtracts.  The caller then adds
   * topk_grad * inv_temperature * grad_scale at the K ids of every row (relax_amd_sparse_row_add).  Rows the step does
   * not read (both masks zero) leave their topk_kl / topk_grad entries untouched: zero them beforehand. */
  const int64_t* topk_ids;              /* [n_tokens, topk_k]; < 0: sentinel (log-prob -inf, no gradient) */
  const float* topk_teacher_log_prob;   /* [n_tokens, topk_k] */
  const int32_t* topk_width;            /* optional [n_tokens]: entries of token t that exist (NULL = topk_k) */
  const int32_t* topk_valid;            /* optional [n_tokens]: union mask, entries k >= topk_valid[t] are masked;
                                           < 0 (or NULL) = no mask for that token */
  int32_t topk_k;                       /* 1 .. RELAX_AMD_FUSED_TOPK_MAX */
  int32_t topk_kl_mode, topk_norm_mode; /* RELAX_AMD_OPD_JSD / _LOW_VAR, RELAX_AMD_OPD_NORM_* */
  int32_t topk_has_clamp;
  float topk_jsd_alpha, topk_min_clamp;
  float* topk_kl;                       /* out [n_tokens] */
  float* topk_grad;                     /* out [n_tokens, topk_k] */
  /* relax_amd_actor_step_fused only: 0 = rows of tokens whose masks are both zero are not read (their log_prob,
   * entropy and distillation outputs are 0, their dlogits rows zeros); 1 = they are scanned like any other row, so
   * that log_prob / entropy / topk_kl hold their true values (what metrics that average over masked tokens too
   * need: opd_per_token_clip_frac, opd_is_clip_frac); their dlogits rows are zeros either way. */
  int32_t read_masked_rows;
} relax_amd_policy_loss_args;

#define RELAX_AMD_FUSED_TOPK_MAX 256

int relax_amd_policy_loss(const relax_amd_policy_loss_args* args, void* stream);

/*
 * Per-sample masked sums: out[i] = sum_t values[t] * mask[t] over sample i's tokens (values NULL = 1).
 * Accumulated in fp64 so integer-valued masks give exact counts.  Replaces loss_mask.sum() per sample
 * (cp_utils.py:140,222) and, with values, one term of sum_of_token (cp_utils.py:156-162).
 */
int relax_amd_segment_sum(const float* values, const float* mask, const int64_t* cu_resp, int64_t n_samples,
                          double* out, void* stream);

/*
 * Group-normalised rewards in input order.  Replaces the group loop of
 * post_process_rewards (relax/utils/utils.py:204-238) and
 * compute_rloo_leave_one_out_rewards (ppo_utils.py:664-705).
 *   rewards, out [n] elements of `dtype` (RELAX_AMD_F32 or RELAX_AMD_F64; arithmetic is done in that type)
 *   group_count [n] out int32: size of the group each sample belongs to (host checks == n_samples_per_prompt)
 */
int relax_amd_group_rewards(const void* rewards, int dtype, const int32_t* group_index, int64_t n, int32_t mode,
                            void* out, int32_t* group_count, void* stream);

/* out[t] = per_sample[i] for every token t of sample i.  Replaces get_grpo_returns (ppo_utils.py:654-661). */
int relax_amd_broadcast_per_sample(const float* per_sample, const int64_t* cu_resp, int64_t n_samples,
                                   float* out, void* stream);

/*
 * Masked whitening with Bessel correction.  Replaces distributed_masked_whiten
 * (relax/utils/distributed_utils.py:98-158) on one rank.
 *   partials [3 * relax_amd_whiten_partials(n)] fp64 workspace
 *   stats    [4] out fp32: sum, sum of squares, mask sum, and 1/sqrt(var+eps)
 */
int64_t relax_amd_whiten_partials(int64_t n);
int relax_amd_masked_whiten(const float* values, const float* mask, int64_t n, int32_t shift_mean, float epsilon,
                            double* partials, float* stats, float* out, void* stream);

/*
 * Per-sequence reverse recurrences over the packed response layout (cu_resp [n_samples+1] int64), fp32 or fp64
 * (dtype RELAX_AMD_F32 / RELAX_AMD_F64 applies to every data pointer of the call).  Each sequence is evaluated in the
 * reference's sequential order, so results are bit-identical to its Python loops.
 *
 * relax_amd_reinforce_pp_returns: get_reinforce_plus_plus_returns (relax/utils/training/ppo_utils.py:708-804, one
 *   context-parallel rank).  G_t = r_t + gamma * G_{t+1}, r_t = -kl_coef * kl[t] on mask != 0 tokens (0 elsewhere,
 *   so masked NaN/inf never enter), rewards[i] added at the last valid token; 0 outside the mask.
 * relax_amd_gae: get_advantages_and_returns / vanilla_gae (ppo_utils.py:846-906, 1026-1047).
 *   delta_t = rewards[t] + gamma * values[t+1] - values[t], A_t = delta_t + gamma*lambd * A_{t+1}, returns = A + values.
 */
int relax_amd_reinforce_pp_returns(const void* kl, const void* mask, const void* rewards, int dtype,
                                   const int64_t* cu_resp, int64_t n_samples, double kl_coef, double gamma,
                                   void* returns, void* stream);
int relax_amd_gae(const void* values, const void* rewards, int dtype, const int64_t* cu_resp, int64_t n_samples,
                  double gamma, double lambd, void* advantages, void* returns, void* stream);

/*
 * REINFORCE++ advantage normaliser on one rank: distributed_masked_normalize (relax/utils/distributed_utils.py:161-213).
 * Population mean / variance (ddof = 0) over mask != 0, out = (x - mean) * rsqrt(max(variance, variance_floor)) on
 * the mask and 0 elsewhere.  stats [3] out (same dtype) = mean, variance, count.
 */
int relax_amd_masked_normalize(const void* values, const void* mask, int dtype, int64_t n, double variance_floor,
                               void* out, void* stats, void* stream);

/*
 * Full-vocab reverse KL(student || teacher) per token and its gradient w.r.t.
 * the student logits.  The K = vocab case of compute_opd_kl's jsd_alpha == 0
 * branch (relax/utils/opd/opd_utils.py:1165-1169) on complete log-softmax rows.
 *   kl, lse_s, lse_t [n_tokens] out
 *   bwd: dstudent = g[t] * grad_scale * (*grad_scale_dev) * p_s * ((log p_s - log p_t) - kl); rows with a zero
 *        incoming gradient are zero-filled without reading
 */
int relax_amd_reverse_kl_fwd(const void* student, const void* teacher, int dtype, int64_t n_tokens, int64_t vocab,
                             int64_t row_stride, float* kl, float* lse_s, float* lse_t, void* stream);
int relax_amd_reverse_kl_bwd(const void* student, const void* teacher, int dtype, int64_t n_tokens, int64_t vocab,
                             int64_t row_stride, const float* kl, const float* lse_s, const float* lse_t,
                             const float* g, float grad_scale, const float* grad_scale_dev, void* dstudent,
                             void* stream);

/*
 * Forward and backward of the reverse KL in one launch, for a reduction whose gradient w.r.t. each token's KL is
 * known before the forward runs: the masked token mean of reduce_opd_loss (relax/utils/opd/opd_utils.py:1355-1365),
 * g[t] = mask[t] / clamp_min(sum mask, 1).  Same outputs as relax_amd_reverse_kl_fwd followed by
 * relax_amd_reverse_kl_bwd (dstudent row stride = row_stride); each workgroup re-reads its two rows out of cache, so
 * HBM moves 3*V*s bytes per token instead of 5*V*s.  Three kernels sit behind it, with bit-identical results: 16-bit
 * rows of the built vocabulary shapes (12 / 15 / 18 / 19 full 16-byte vectors per thread of 1024 threads plus a
 * partial one, or 16 / 20 exactly; the default kernel also 6 / 7 / 24 / 30 / 31 plus a partial one and 8 / 32 exactly) are shared by eight
 * one-shot workgroups that keep both rows' shares on chip, so each row is read once (the default), or, after
 * relax_amd_set_kernel_choice(RELAX_AMD_KERNEL_RESIDENT), kept as the student row in the registers of one persistent
 * workgroup that streams the teacher row past it twice; other rows, and every row after
 * relax_amd_set_kernel_choice(RELAX_AMD_KERNEL_TWO_WALK), walk both rows twice.
 */
int relax_amd_reverse_kl_step_fused(const void* student, const void* teacher, int dtype, int64_t n_tokens,
                                    int64_t vocab, int64_t row_stride, const float* g, float grad_scale, float* kl,
                                    float* lse_s, float* lse_t, void* dstudent, void* stream);

/*
 * Log-prob + entropy with a vocabulary keep mask: the log_prob_keep_mask branch of
 * _VocabParallelLogProbEntropy.forward / .backward (relax/utils/training/ppo_utils.py:546-567, 597-629).  The
 * log-prob's softmax runs over the entries whose mask byte is non-zero plus the target; the entropy over the whole row.
 *   keep_mask  uint8 [n_tokens, vocab] indexed by token (row stride keep_stride >= vocab)
 *   lse_kept   fp32 [n_tokens] out: log-sum-exp over kept entries (needed by the backward)
 *   entropy, lse_full, spx   fp32 [n_tokens] out, may be NULL when no entropy is wanted
 * bwd: dlogits = g_lp*(onehot - keep'*p_kept)/T + g_ent*p_full*(spx - x/T)/T, keep' = keep or target; every row
 *      is written once.
 */
int relax_amd_logprob_entropy_masked_fwd(const void* logits, int dtype, int64_t n_tokens, int64_t vocab,
                                         int64_t row_stride, const int32_t* row_ids, const int64_t* targets,
                                         const uint8_t* keep_mask, int64_t keep_stride, float inv_temperature,
                                         float* log_prob, float* entropy, float* lse_kept, float* lse_full, float* spx,
                                         void* stream);
int relax_amd_logprob_entropy_masked_bwd(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                                         int64_t row_stride, const int32_t* token_of_row, const int64_t* targets,
                                         const uint8_t* keep_mask, int64_t keep_stride, const float* lse_kept,
                                         const float* lse_full, const float* spx, const float* g_lp,
                                         const float* g_ent, float grad_scale, float inv_temperature, void* dlogits,
                                         int64_t d_row_stride, void* stream);

/*
 * Log-probs of K given vocabulary ids per token: compute_log_probs_on_topk_token_ids
 * (relax/utils/opd/opd_utils.py:1022-1094) on one rank.
 *   topk_ids      int64 [n_tokens, k]; ids < 0 are sentinels (-inf out, no gradient), ids >= vocab read as a zero
 *                 logit (the reference's fill for ids outside the rank's vocabulary slice)
 *   row_ids       int32 [n_tokens] logits row of each token, or NULL (row t = token t)
 *   lse_in        fp32 [n_tokens] log-sum-exp of each token's row (as written by relax_amd_logprob_entropy_fwd), or
 *                 NULL: the kernel scans the row itself and writes lse_out (if not NULL)
 *   topk_log_prob fp32 [n_tokens, k] out = logits[row, id] * inv_temperature - lse
 * bwd: dlogits[row, v] = inv_temperature * ( sum_k g[t,k] * [v == id_k] - p[v] * sum_{k: id_k >= 0} g[t,k] ),
 *   every row written once (rows with token_of_row < 0 or an all-zero g are zero-filled without a read).
 */
int relax_amd_topk_logprob_fwd(const void* logits, int dtype, int64_t n_tokens, int64_t vocab, int64_t row_stride,
                               const int32_t* row_ids, const int64_t* topk_ids, int64_t k, float inv_temperature,
                               const float* lse_in, float* topk_log_prob, float* lse_out, void* stream);
int relax_amd_topk_logprob_bwd(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                               const int32_t* token_of_row, const int64_t* topk_ids, int64_t k, float inv_temperature,
                               const float* lse, const float* g, void* dlogits, int64_t d_stride, void* stream);

/*
 * Per-token distillation signal on [n_rows, k] top-K log-probs: compute_opd_kl_topk / compute_opd_kl
 * (relax/utils/opd/opd_utils.py:1097-1228).
 *   mask          uint8 [n_rows, k] (non-zero = valid) for the union path's padded rows, or NULL.  With a mask the
 *                 padded entries are excluded and, as in the reference, the tail bin is cut off as well.
 *   kl_mode       RELAX_AMD_OPD_JSD (jsd_alpha in [0, 1]) or RELAX_AMD_OPD_LOW_VAR
 *   norm_mode     RELAX_AMD_OPD_NORM_* (JSD family only)
 *   has_clamp / log_prob_min_clamp   clamp both inputs from below first (opd_log_prob_min_clamp)
 *   k             1..2048
 * bwd: d_student_lp[r, j] = g[r] * d kl[r] / d student_lp[r, j]  (the teacher is detached)
 */
int relax_amd_opd_kl_topk_fwd(const float* student_lp, const float* teacher_lp, const uint8_t* mask, int64_t n_rows,
                              int64_t k, int kl_mode, int norm_mode, float jsd_alpha, int has_clamp,
                              float log_prob_min_clamp, float* kl, void* stream);
int relax_amd_opd_kl_topk_bwd(const float* student_lp, const float* teacher_lp, const uint8_t* mask, int64_t n_rows,
                              int64_t k, int kl_mode, int norm_mode, float jsd_alpha, int has_clamp,
                              float log_prob_min_clamp, const float* g, float* d_student_lp, void* stream);

/*
 * dlogits[row_ids[t], ids[t, j]] += values[t, j] * scale for j < k, and dlogits[row_ids[t], targets[t]] +=
 * target_values[t] * scale: the sparse part of the gradient of gathered log-probs (the scatter of
 * compute_log_probs_on_topk_token_ids' backward, relax/utils/opd/opd_utils.py:1022-1094) when its dense part, a
 * multiple of the row's softmax, has been folded into the dlogits launch of the log-prob backward.  Ids outside
 * [0, vocab), zero values and tokens with a negative row id are skipped; targets / target_values may be NULL;
 * row_ids NULL = row t.
 */
int relax_amd_sparse_row_add(void* dlogits, int dtype, int64_t n_tokens, int64_t vocab, int64_t row_stride,
                             const int32_t* row_ids, const int64_t* ids, const float* values, int64_t k,
                             const int64_t* targets, const float* target_values, float scale, void* stream);

/*
 * The k largest logits of each token's row and their vocabulary ids, largest first: torch.topk(logits_chunk, k=k,
 * dim=-1) of get_log_probs_and_entropy (relax/backends/megatron/loss.py:434-436), for every response row in one
 * launch.  NaN orders above +inf as in torch.topk; which of several equal values at the k-th place is returned is
 * unspecified there and here.
 *   row_ids  int32 [n_tokens] logits row of each token, or NULL (row t = token t)
 *   values   fp32 [n_tokens, k] out (the logits as fp32), or NULL
 *   indices  int64 [n_tokens, k] out
 *   workspace n_tokens bytes of device memory (one flag per row: rows with long runs of equal values take a second,
 *            general kernel)
 * 1 <= k <= 512 and vocab <= 1000000, otherwise RELAX_AMD_EUNSUPPORTED.
 */
int relax_amd_topk_rows(const void* logits, int dtype, int64_t n_tokens, int64_t vocab, int64_t row_stride,
                        const int32_t* row_ids, int k, float* values, int64_t* indices, uint8_t* workspace,
                        void* stream);

/*
 * relax_amd_logprob_entropy_fwd and relax_amd_topk_rows over the same response rows from one read of the logits: what
 * get_log_probs_and_entropy(..., with_topk=True) computes per sample (relax/backends/megatron/loss.py:373-446: the
 * log-probs / entropy of the response tokens and torch.topk of the same logits rows).  Arguments as in those two
 * functions; log_prob / entropy / lse / spx are bit-identical to relax_amd_logprob_entropy_fwd's, values / indices
 * follow relax_amd_topk_rows' contract (the selection does not depend on the temperature).  Rows that are not whole
 * 16-byte vectors in groups of eight, or too short for the forward scan's 1024-thread workgroups (fewer than 7168
 * vectors), run the two passes one after the other.
 */
int relax_amd_logprob_entropy_topk_fwd(const void* logits, int dtype, int64_t n_tokens, int64_t vocab,
                                       int64_t row_stride, const int32_t* row_ids, const int64_t* targets,
                                       float inv_temperature, int k, float* log_prob, float* entropy, float* lse,
                                       float* spx, float* values, int64_t* indices, uint8_t* workspace, void* stream);

/*
 * Fused actor step: log-prob + entropy forward, the per-token terms of relax_amd_policy_loss and the dlogits backward
 * in one launch.  Each workgroup scans its row, derives the token's gradient constants and immediately walks the row
 * again to emit dlogits; the second walk is served by the L2 / memory-side cache, so HBM sees one read and one write
 * per row.  Replaces, for one micro-batch, _VocabParallelLogProbEntropy.forward + .backward (ppo_utils.py:481-629)
 * fused with the per-token part of policy_loss_function (loss.py:961-1100).  Available when d loss / d log_prob of a
 * token depends on that token only: every loss kind except GSPO, no OPSM (those return RELAX_AMD_EUNSUPPORTED).
 * Its log-probs / entropy are bit-identical to relax_amd_logprob_entropy_fwd's on the same rows.
 *   loss        the same argument block relax_amd_policy_loss takes; its log_prob / entropy inputs are ignored
 *               (they are produced here), coef_log_prob / coef_entropy are written; metrics are NOT produced: call
 *               relax_amd_policy_loss afterwards with log_prob / entropy set to this call's outputs
 *   sample_ids  [n_tokens] int32 sample of each token (needed with per-sample denominators)
 *   grad_scale  host scalar folded into dlogits (the upstream gradient the caller expects, normally 1)
 *   log_prob, entropy, lse, spx  [n_tokens] out; tokens whose masks are both zero get zeros (their row is not read)
 *               unless loss->read_masked_rows is set
 *   dlogits     [n_rows, vocab] out, every row written (zero rows where token_of_row < 0 or the coefficients vanish)
 * With loss->topk_ids set the step also evaluates the top-K distillation signal of every row it reads (see the
 * argument block); the caller adds the K one-hot parts of its gradient with relax_amd_sparse_row_add afterwards.
 * Three kernels sit behind this entry point and are chosen by row length and element type, all with the same
 * results bit for bit: one-shot workgroups that share each row (one read and one write of HBM per row; 16-bit rows of
 * 28680 .. 32768, 49160 .. 53248, 57352 .. 65536, 100352 .. 163840, 196616 .. 204800 and 245768 .. 262144 entries
 * (the last two ranges keep part of the row in LDS), fp32 rows of 28676 .. 32768, 49156 .. 53248,
 * 61444 .. 65536 and, part of the row in LDS, 100352 .. 163840 and 245764 .. 249856 entries, in the built shapes: the default where built, see
 * relax_amd_set_kernel_choice for the ring in device memory it exchanges partial sums through), a persistent
 * register-resident one (the same traffic, the same shapes) and a two-walk one for everything
 * else; relax_amd_set_kernel_choice(RELAX_AMD_KERNEL_RESIDENT / RELAX_AMD_KERNEL_TWO_WALK) forces the second / third.
 */
int relax_amd_actor_step_fused(const void* logits, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                               const int32_t* token_of_row, const int32_t* sample_ids, const int64_t* targets,
                               float inv_temperature, const relax_amd_policy_loss_args* loss, float grad_scale,
                               float* log_prob, float* entropy, float* lse, float* spx, void* dlogits,
                               int64_t d_row_stride, void* stream);
/* data[row, :] *= *factor_dev in place; returns immediately on the device when the factor is 1 to within 2^-20 (a
 * product of fp32 factors that equals the assumed scale mathematically may differ from it in the last bits).  Lets an
 * autograd backward apply upstream / grad_scale when the upstream scalar turns out to differ from the grad_scale
 * assumed above, without a host read. */
int relax_amd_scale_rows_inplace(void* data, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                 const float* factor_dev, void* stream);

/*
 * Fused LM-head projection + log-prob / entropy: logits = hidden @ weight^T are formed tile by tile on the bf16
 * matrix cores and reduced in registers; the [n_tokens, vocab] logits are never written.  Replaces the
 * deferred-LM-head branch of get_log_probs_and_entropy (relax/backends/megatron/loss.py:391-419: per sub-chunk
 * lm_head_forward -> .float() -> /T -> calculate_log_probs_and_entropy) and additionally returns the entropy.
 *   hidden [n_tokens, hidden_size] bf16 (row stride h_stride), weight [vocab, hidden_size] bf16 (row stride w_stride)
 *   hidden_size must be a multiple of 128; rows 16-byte aligned
 *   workspace  relax_amd_lmhead_workspace_bytes(n_tokens) bytes of device memory
 */
int64_t relax_amd_lmhead_workspace_bytes(int64_t n_tokens);
int relax_amd_lmhead_logprob_fwd(const void* hidden, const void* weight, int dtype, int64_t n_tokens,
                                 int64_t hidden_size, int64_t vocab, int64_t h_stride, int64_t w_stride,
                                 const int64_t* targets, float inv_temperature, void* workspace, float* log_prob,
                                 float* entropy, float* lse, float* spx, void* stream);
/*
 * The same forward pass for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Identical to
 * relax_amd_lmhead_logprob_fwd except that the workspace is a fixed array inside the library (one copy per GPU,
 * RELAX_AMD_LMHEAD_STATIC_SCRATCH_BYTES, held until the process ends), so the call allocates and frees nothing.
 * n_tokens above RELAX_AMD_LMHEAD_STATIC_MAX_TOKENS returns RELAX_AMD_EUNSUPPORTED.  All calls on one GPU share
 * that GPU's array: calls that overlap in time on one GPU (different streams or threads) race; serialise them.
 * The first call on a device looks the array's address up (hipGetSymbolAddress); make it outside graph capture.
 */
#define RELAX_AMD_LMHEAD_STATIC_MAX_TOKENS 32768
#define RELAX_AMD_LMHEAD_STATIC_SCRATCH_BYTES (25 * 4 * RELAX_AMD_LMHEAD_STATIC_MAX_TOKENS)
int relax_amd_lmhead_logprob_fwd_static(const void* hidden, const void* weight, int dtype, int64_t n_tokens,
                                        int64_t hidden_size, int64_t vocab, int64_t h_stride, int64_t w_stride,
                                        const int64_t* targets, float inv_temperature, float* log_prob,
                                        float* entropy, float* lse, float* spx, void* stream);
/*
 * Backward helper of the fused LM head: recomputes the logits of n_tokens rows on the matrix cores and writes the
 * gradient w.r.t. the logits, transposed and in bf16:
 *   d_t[v, n] = inv_T * ( g_lp[n]*(onehot(target[n]) - p) + g_ent[n] * p * (spx[n] - x) ),  p = exp(x - lse[n])
 * (autograd through F.linear + _VocabParallelLogProbEntropy.backward, ppo_utils.py:591-629).  The caller contracts
 * d_t with weight (dhidden) and hidden (dweight) by plain GEMMs, slab by slab, so only one [vocab, n_tokens] slab
 * exists at a time.  d_t has row stride d_stride >= n_tokens.
 */
int relax_amd_lmhead_dlogits_t(const void* hidden, const void* weight, int dtype, int64_t n_tokens,
                               int64_t hidden_size, int64_t vocab, int64_t h_stride, int64_t w_stride,
                               const int64_t* targets, const float* lse, const float* spx, const float* g_lp,
                               const float* g_ent, const float* grad_scale_dev, float inv_temperature, void* d_t,
                               int64_t d_stride, void* stream);

/*
 * The two contractions of the gradient slab d_t [vocab, n_tokens] (bf16, token contiguous: what
 * relax_amd_lmhead_dlogits_t / relax_amd_lmhead_dlogits_from_logits_t produce) that autograd through F.linear performs
 * in the deferred-LM-head branch (relax/backends/megatron/loss.py:391-419, model.py:151-166), on the matrix cores:
 *   relax_amd_lmhead_dhidden:  d_hidden[n, h] = sum_v d_t[v, n] * weight[v, h]
 *   relax_amd_lmhead_dweight:  d_weight[v, h] = sum_n d_t[v, n] * hidden[n, h]
 * Operands are read in the layouts they have (no transposed copies).  Reads past an operand's end are clamped and
 * rely on zeros in d_t: d_t must be allocated with d_rows >= ceil128(vocab) rows of d_stride >= ceil128(n_tokens)
 * elements, holding zeros in rows >= vocab and columns >= n_tokens up to those rounded sizes (the producers above
 * never write there, so clearing the padding once after allocation is enough).  hidden_size and all row strides must
 * be multiples of 8, bases 16-byte aligned.
 *   out_mode  RELAX_AMD_GEMM_OUT_BF16: out is bf16; _F32: out is fp32; _F32_ACCUMULATE: out (fp32) += the product
 *             (accumulation of d_weight over several slabs of tokens)
 */
enum { RELAX_AMD_GEMM_OUT_BF16 = 0, RELAX_AMD_GEMM_OUT_F32 = 1, RELAX_AMD_GEMM_OUT_F32_ACCUMULATE = 2 };
int relax_amd_lmhead_dhidden(const void* d_t, int64_t d_rows, int64_t d_stride, const void* weight, int64_t w_stride,
                             int64_t n_tokens, int64_t hidden_size, int64_t vocab, void* d_hidden, int64_t dh_stride,
                             int out_mode, void* stream);
int relax_amd_lmhead_dweight(const void* d_t, int64_t d_stride, const void* hidden, int64_t h_stride,
                             int64_t n_tokens, int64_t hidden_size, int64_t vocab, void* d_weight, int64_t dw_stride,
                             int out_mode, void* stream);

/*
 * The same forward pass that also keeps the logits: logits_t [vocab, l_stride] bf16 (token contiguous, l_stride >=
 * n_tokens) receives bf16(hidden @ weight^T), and the softmax statistics and the target logit are taken from those
 * rounded values -- the reference's own numerics, whose F.linear runs in the weight dtype before .float()
 * (relax/backends/megatron/loss.py:405-409).  For callers that would rather spend vocab * n_tokens * 2 bytes of HBM
 * than recompute the projection in the backward pass (the reference's non-deferred path keeps the logits too).
 */
int relax_amd_lmhead_logprob_fwd_keep(const void* hidden, const void* weight, int dtype, int64_t n_tokens,
                                      int64_t hidden_size, int64_t vocab, int64_t h_stride, int64_t w_stride,
                                      const int64_t* targets, float inv_temperature, void* workspace, float* log_prob,
                                      float* entropy, float* lse, float* spx, void* logits_t, int64_t l_stride,
                                      void* stream);
/*
 * Backward from kept logits: overwrites logits_t in place with the d_t of relax_amd_lmhead_dlogits_t (same formula,
 * x = the stored bf16 logit), one read and one write of the slab instead of a second projection
 * (_VocabParallelLogProbEntropy.backward, ppo_utils.py:591-629, applied to the stored logits).
 * l_stride must be a multiple of 8 and logits_t 16-byte aligned.  Columns n_tokens .. ceil8(n_tokens) - 1 are written
 * as zeros and later columns are not touched, so a slab whose padding was cleared once can go to
 * relax_amd_lmhead_dhidden / relax_amd_lmhead_dweight as it is (a slab reused for FEWER tokens than a call before
 * still holds that call's values in columns ceil8(n_tokens) .. and needs them cleared up to ceil128(n_tokens)).
 */
int relax_amd_lmhead_dlogits_from_logits_t(void* logits_t, int64_t n_tokens, int64_t vocab, int64_t l_stride,
                                           const int64_t* targets, const float* lse, const float* spx,
                                           const float* g_lp, const float* g_ent, const float* grad_scale_dev,
                                           float inv_temperature, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* RELAX_AMD_H */
