// Per-token policy-loss arithmetic shared by the stand-alone policy-loss kernel and the fused actor-step kernel, so
// both produce the same loss terms and the same d loss / d log_prob coefficients.
//
// Gradient conventions reproduced from autograd over the reference's torch ops
// (relax/utils/training/ppo_utils.py:100-396, relax/backends/megatron/loss.py:741-769, 961-1134):
//   PPO-clip   d/dlp = -A*r when r is inside [1-eps_lo, 1+eps_hi] or the unclipped branch is strictly larger, else 0
//   dual clip  A<0 and -c*A < clipped loss: 0; tie: half
//   CISPO      -coef*A (coef, A detached);  RLOO  -A;  SAPO  -A*4*s*(1-s)*r  (s = sigmoid(tau*(r-1)))
//   k1: 1   k2: d   k3 / low_var: 1-exp(-d)  (low_var: 0 outside the [-10,10] clamp)
//   unbiased KL multiplies by ratio = exp(lp-old) and adds ratio*kl (the ratio is not detached, loss.py:1091)
#pragma once

#include "device_utils.h"
#include "relax_amd.h"

namespace relax_amd {

struct TokenTerms {
  float pg, clipfrac, ppo_kl, dpg_dlp, dpg_dkl;
};

// One token of compute_policy_loss / compute_cispo_loss / compute_rloo_loss / compute_sapo_loss.
// `kl` is old - lp (token-level) or the sequence KL (GSPO).  dpg_dlp is the derivative through a token-level kl
// (d kl / d lp = -1) plus any direct lp dependence; dpg_dkl is the derivative w.r.t. kl itself (used by GSPO).
__device__ __forceinline__ TokenTerms token_loss(int kind, float lp, float kl, float adv, float eps_lo, float eps_hi,
                                                 float eps_c, float tau_pos, float tau_neg) {
  TokenTerms t;
  t.ppo_kl = kl;
  const float r = expf(-kl);
  if (kind == RELAX_AMD_LOSS_CISPO) {
    const float hi = 1.0f + eps_hi, lo = 1.0f - eps_lo;
    const float coef = adv >= 0.f ? fminf(r, hi) : fmaxf(r, lo);
    t.pg = -(coef * adv * lp);
    t.clipfrac = ((adv >= 0.f && r > hi) ? 1.f : 0.f) + ((adv < 0.f && r < lo) ? 1.f : 0.f);
    t.dpg_dlp = -(coef * adv);
    t.dpg_dkl = 0.f;
    return t;
  }
  if (kind == RELAX_AMD_LOSS_RLOO) {
    t.pg = -(adv * lp);
    t.clipfrac = 0.f;
    t.dpg_dlp = -adv;
    t.dpg_dkl = 0.f;
    return t;
  }
  if (kind == RELAX_AMD_LOSS_SAPO) {
    const float tau = adv > 0.f ? tau_pos : tau_neg;
    const float s = 1.0f / (1.0f + expf(-tau * (r - 1.0f)));
    t.pg = -((4.0f / tau) * s * adv);
    t.clipfrac = (4.0f * s * (1.0f - s)) < 0.9f ? 1.f : 0.f;
    // d pg / d r = -(4/tau)*adv*tau*s*(1-s);  d r / d kl = -r
    t.dpg_dkl = 4.0f * adv * s * (1.0f - s) * r;
    t.dpg_dlp = -t.dpg_dkl;
    return t;
  }
  // PPO clip (also the per-token function GSPO applies to the sequence KL)
  const float lo = 1.0f - eps_lo, hi = 1.0f + eps_hi;
  const float l1 = -r * adv;
  const float rc = fminf(fmaxf(r, lo), hi);
  const float l2 = -rc * adv;
  float loss = fmaxf(l1, l2);
  t.clipfrac = l2 > l1 ? 1.f : 0.f;
  const bool inside = (r >= lo) && (r <= hi);
  float dl_dr = (inside || l1 > l2) ? -adv : 0.f;  // ties outside the range only occur at adv == 0
  if (eps_c > 0.f && adv < 0.f) {
    const float l3 = -eps_c * adv;
    if (l3 < loss) {
      loss = l3;
      dl_dr = 0.f;
    } else if (l3 == loss) {
      dl_dr *= 0.5f;
    }
  }
  t.pg = loss;
  t.dpg_dkl = -dl_dr * r;  // d r / d kl = -r
  t.dpg_dlp = dl_dr * r;
  return t;
}

__device__ __forceinline__ void kl_term(int kind, float lp, float ref, float& kl, float& dkl_dlp) {
  const float d = lp - ref;
  if (kind == RELAX_AMD_KL_K1) {
    kl = d;
    dkl_dlp = 1.f;
  } else if (kind == RELAX_AMD_KL_K2) {
    kl = d * d / 2.0f;
    dkl_dlp = d;
  } else {
    const float e = expf(-d);
    kl = e - 1.0f - (-d);
    dkl_dlp = 1.0f - e;
  }
}


// NULL when the caller's struct_size covers this library's relax_amd_policy_loss_args, else the message to report.
// Checked before any other field is read: a client built against a shorter layout would otherwise have the bytes
// behind its struct taken for device pointers.
const char* policy_loss_args_size_error(const relax_amd_policy_loss_args* a);

// Host-side check of the optional distillation fields; NULL when they are consistent.
inline const char* distill_args_error(const relax_amd_policy_loss_args& a) {
  if (!a.distill_teacher_log_prob) return nullptr;
  if (!a.extra_coef_log_prob) return "distill_teacher_log_prob needs extra_coef_log_prob (the signal's weights)";
  if (a.distill_kl_kind != RELAX_AMD_KL_K1 && a.distill_kl_kind != RELAX_AMD_KL_K3)
    return "distill_kl_kind must be RELAX_AMD_KL_K1 or RELAX_AMD_KL_K3";
  return nullptr;
}

struct TokenResult {
  float metric[RELAX_AMD_NUM_METRICS];  // this token's masked contribution to every per-sample sum
  float pg, clipfrac, ppo_kl, kl;       // un-masked per-token values
  float coef_lp, coef_ent;              // d loss / d log_prob (token-local part), d loss / d entropy
  float g_seq;                          // GSPO: w_t * d pg_t / d kl_i, summed per sequence by the caller
};

// Per-token inputs of the loss, fetched ahead of time so their latency can hide behind other work.
struct TokenInputs {
  float old_lp, ref_lp, train_lp, rollout_lp, adv, m, mp;
  float extra_lp;    // caller-supplied addition to d loss / d log_prob (0 when there is none)
  float teacher_lp;  // teacher log-prob of the sampled-token distillation signal (when that is configured)
  bool has_old, has_train;
};

__device__ __forceinline__ TokenInputs load_token_inputs(const relax_amd_policy_loss_args& a, int64_t t) {
  TokenInputs in;
  in.has_old = a.old_log_prob != nullptr;
  in.has_train = a.train_log_prob != nullptr;
  in.old_lp = in.has_old ? a.old_log_prob[t] : 0.f;
  in.ref_lp = (a.kl_kind != RELAX_AMD_KL_NONE) ? a.ref_log_prob[t] : 0.f;
  in.train_lp = in.has_train ? a.train_log_prob[t] : 0.f;
  in.rollout_lp = a.rollout_log_prob ? a.rollout_log_prob[t] : 0.f;
  in.adv = a.advantages[t];
  in.m = a.loss_mask[t];
  in.mp = a.pg_loss_mask ? a.pg_loss_mask[t] : in.m;
  in.extra_lp = a.extra_coef_log_prob ? a.extra_coef_log_prob[t] : 0.f;
  in.teacher_lp = a.distill_teacher_log_prob ? a.distill_teacher_log_prob[t] : 0.f;
  return in;
}

// All per-token terms of policy_loss_function for one token given its current log-prob and entropy.
// `den` / `pg_den` are the sample's divisors; `seq_kl` the sequence KL (GSPO / OPSM only).
__device__ __forceinline__ TokenResult token_terms(const relax_amd_policy_loss_args& a, const TokenInputs& in, float lp,
                                                   float entropy, bool gspo, float seq_kl, float den, float pg_den) {
  TokenResult o;
#pragma unroll
  for (int k = 0; k < RELAX_AMD_NUM_METRICS; ++k) o.metric[k] = 0.f;
  const int kind = gspo ? RELAX_AMD_LOSS_PPO : a.loss_kind;
  const float old = in.has_old ? in.old_lp : lp;
  const float adv = in.adv;
  const float m = in.m;
  const float mp = in.mp;
  const float kl_in = gspo ? seq_kl : (old - lp);
  TokenTerms tt = token_loss(kind, lp, kl_in, adv, a.eps_clip, a.eps_clip_high, a.eps_clip_c, a.tau_pos, a.tau_neg);
  float w = 1.0f;  // multiplicative, gradient-free weights on pg_loss
  float drop = 0.f;
  if (a.use_opsm) {
    drop = (adv < 0.f && seq_kl > a.opsm_delta) ? 1.f : 0.f;
    w *= 1.0f - drop;
  }
  float tis = 0.f, log_ratio = 0.f, tis_w = 1.f;
  const bool have_tis = (a.use_tis || a.mismatch_metrics) && a.rollout_log_prob;
  if (have_tis) {
    log_ratio = (in.has_train ? in.train_lp : lp) - in.rollout_lp;
    tis = expf(log_ratio);
    tis_w = fminf(fmaxf(tis, a.tis_lo), a.tis_hi);
    w *= tis_w;
  }
  o.pg = tt.pg * w;
  o.clipfrac = tt.clipfrac;
  o.ppo_kl = tt.ppo_kl;
  o.kl = 0.f;
  o.coef_lp = (mp / pg_den) * w * (gspo ? 0.f : tt.dpg_dlp);
  o.g_seq = gspo ? (mp / pg_den) * w * tt.dpg_dkl : 0.f;
  o.coef_ent = -a.entropy_coef * (m / den);

  o.metric[RELAX_AMD_M_PG_LOSS] = o.pg * mp;
  o.metric[RELAX_AMD_M_CLIPFRAC] = tt.clipfrac * m;
  o.metric[RELAX_AMD_M_PPO_KL] = tt.ppo_kl * m;
  o.metric[RELAX_AMD_M_MASK_SUM] = m;
  o.metric[RELAX_AMD_M_ENTROPY] = entropy * m;
  if (a.kl_kind != RELAX_AMD_KL_NONE) {
    float kl, dkl;
    kl_term(a.kl_kind, lp, in.ref_lp, kl, dkl);
    if (a.unbiased_kl) {
      const float ratio = expf(lp - old);
      dkl = ratio * dkl + ratio * kl;  // ratio carries gradient (d ratio / d lp = ratio)
      kl = ratio * kl;
    }
    if (a.kl_kind == RELAX_AMD_KL_LOW_VAR) {
      if (kl < -10.f || kl > 10.f) dkl = 0.f;
      kl = fminf(fmaxf(kl, -10.f), 10.f);
    }
    o.kl = kl;
    o.metric[RELAX_AMD_M_KL_LOSS] = kl * m;
    o.coef_lp += a.kl_coef * (m / den) * dkl;
  }
  float extra = in.extra_lp;
  if (a.topk_ids) extra = 0.f;  // the weight of the top-K distillation signal, which the fused step evaluates itself
  if (a.distill_teacher_log_prob) {
    // extra_lp is the weight of this token's distillation signal in the loss; the signal's own derivative follows
    // the chain clamp_min -> estimator -> clamp(max = token clip) -> x min(ratio, clip) with the ratio detached
    float s = lp, t = in.teacher_lp, pass = 1.f;
    if (a.distill_min_clamp == a.distill_min_clamp) {  // set (not NaN)
      if (s < a.distill_min_clamp) {
        s = a.distill_min_clamp;
        pass = 0.f;
      }
      t = fmaxf(t, a.distill_min_clamp);
    }
    float sig, dsig;
    kl_term(a.distill_kl_kind, s, t, sig, dsig);
    if (a.distill_token_clip == a.distill_token_clip && sig > a.distill_token_clip) pass = 0.f;
    if (a.distill_is_clip == a.distill_is_clip) pass *= fminf(expf(lp - old), a.distill_is_clip);
    extra *= pass * dsig;
  }
  o.coef_lp += extra;
  if (a.rollout_log_prob) {
    const float roll = in.rollout_lp;
    float side = lp;
    if (a.abs_diff_from_old == 1) side = old;
    else if (a.abs_diff_from_old == 0 && in.has_train) side = in.train_lp;
    o.metric[RELAX_AMD_M_LOGPROB_ABS_DIFF] = fabsf(side - roll) * m;
    o.metric[RELAX_AMD_M_PROB_ABS_DIFF] = fabsf(expf(side) - expf(roll)) * m;
  }
  if (have_tis) {
    o.metric[RELAX_AMD_M_OIS] = expf(-tt.ppo_kl) * m;
    o.metric[RELAX_AMD_M_TIS] = tis * m;
    o.metric[RELAX_AMD_M_TIS_CLIPFRAC] = (tis_w != tis ? 1.f : 0.f) * m;
    o.metric[RELAX_AMD_M_TIS_ABS] = fabsf(tis - 1.0f) * m;
    o.metric[RELAX_AMD_M_MISMATCH_KL] = (-log_ratio) * m;
    o.metric[RELAX_AMD_M_MISMATCH_K3] = (tis - log_ratio - 1.0f) * m;
  }
  o.metric[RELAX_AMD_M_OPSM_CLIPFRAC] = drop;
  if (m == 0.f && mp == 0.f) {
    // A fully masked token is selected out rather than multiplied by its zero mask, so a non-finite value sitting at
    // a padded position cannot reach any sum or gradient: the mask-safe reducer the reference wraps around the
    // REINFORCE++ estimators (loss.py:804-821), applied to every estimator here (finite inputs give the same result).
#pragma unroll
    for (int k = 0; k < RELAX_AMD_NUM_METRICS; ++k)
      if (k != RELAX_AMD_M_OPSM_CLIPFRAC) o.metric[k] = 0.f;
    o.coef_lp = 0.f;
    o.coef_ent = 0.f;
    o.g_seq = 0.f;
  }
  return o;
}

}  // namespace relax_amd
