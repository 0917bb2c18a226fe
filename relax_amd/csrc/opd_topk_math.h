// Per-token KL family of the top-K distillation signal on one row of [K] (student, teacher) log-prob pairs, computed
// by one wave: compute_opd_kl_topk / compute_opd_kl (relax/utils/opd/opd_utils.py:1097-1228) with tail bin,
// renormalisation, truncation, the lower clamp and the union path's padding mask.  Shared by the stand-alone [R, K]
// kernels and by the fused actor step, which evaluates the term next to a row's log-sum-exp, so both return the same
// bits for the same inputs.
#pragma once

#include <cmath>
#include <cstdint>

#include "device_utils.h"
#include "relax_amd.h"

namespace relax_amd {

struct OpdParams {
  int mode;       // RELAX_AMD_OPD_JSD family (alpha = 0: reverse KL, 1: forward KL) or RELAX_AMD_OPD_LOW_VAR
  int norm;       // RELAX_AMD_OPD_NORM_*
  float alpha;
  int has_clamp;
  float clamp;
};

// log-sum-exp over the lanes' strided values (−inf entries contribute nothing; all −inf gives −inf)
__device__ __forceinline__ float row_logsumexp(const float* v, int n, int lane) {
  float m = -INFINITY;
  for (int k = lane; k < n; k += kWave) m = fmaxf(m, v[k]);
  m = wave_max(m);
  if (m == -INFINITY) return -INFINITY;
  float s = 0.f;
  for (int k = lane; k < n; k += kWave) s += expf(v[k] - m);
  s = wave_sum(s);
  return m + logf(s);
}

// term of one (s', t') entry and its derivative w.r.t. s'
__device__ __forceinline__ void opd_entry(float s, float t, float alpha, float log_1ma, float log_a, float& term,
                                          float& dterm) {
  if (alpha == 0.f) {
    const float p = expf(s);
    term = p * (s - t);
    dterm = p * (s - t + 1.f);
  } else if (alpha == 1.f) {
    const float q = expf(t);
    term = q * (t - s);
    dterm = -q;
  } else {
    const float u = s + log_1ma, w = t + log_a;
    const float hi = fmaxf(u, w);
    const float m = (hi == -INFINITY) ? -INFINITY : hi + logf(expf(u - hi) + expf(w - hi));
    const float p = expf(s), q = expf(t);
    term = (1.f - alpha) * (p * (s - m)) + alpha * (q * (t - m));
    dterm = (1.f - alpha) * p * (s - m);
  }
}

// The row's KL (returned in every lane) and, with BWD, d KL / d student entry for every k.
//   load_s(k), load_t(k): the row's raw student / teacher log-probs;  valid(k): the union mask (called only when
//   has_mask);  store_d(k, dk, nonzero): receives each entry's derivative (dk is meaningless when !nonzero: the entry
//   is masked or clamped and gets no gradient).
//   sv, tv: k_ids floats of LDS each, private to the wave.  Every lane re-reads only the entries it staged itself
//   (k = lane, lane + 64, ...), so no barrier is needed; store_d(k, ...) is the last use of sv[k] / tv[k] and may
//   overwrite them.
template <bool BWD, typename LoadS, typename LoadT, typename Valid, typename StoreD>
__device__ __forceinline__ float opd_kl_row(int k_ids, bool has_mask, const OpdParams& p, int lane, float* sv,
                                            float* tv, LoadS&& load_s, LoadT&& load_t, Valid&& valid,
                                            StoreD&& store_d) {
  for (int k = lane; k < k_ids; k += kWave) {
    float a = load_s(k), b = load_t(k);
    if (p.has_clamp) {
      a = fmaxf(a, p.clamp);  // NaN stays out of scope: log-probs are never NaN on entry
      b = fmaxf(b, p.clamp);
    }
    if (has_mask && !valid(k)) a = b = -INFINITY;
    sv[k] = a;
    tv[k] = b;
  }
  if (p.mode == RELAX_AMD_OPD_LOW_VAR) {
    float acc = 0.f;
    for (int k = lane; k < k_ids; k += kWave) {
      const bool ok = !has_mask || valid(k);
      const float d = sv[k] - tv[k];
      const float e = expf(-d);
      if (ok) acc += e - 1.f + d;
      if (BWD) {
        const bool pass = !p.has_clamp || load_s(k) >= p.clamp;
        store_d(k, 1.f - e, ok && pass);
      }
    }
    return wave_sum(acc);
  }
  const float ls = row_logsumexp(sv, k_ids, lane), lt = row_logsumexp(tv, k_ids, lane);
  float shift_s = 0.f, shift_t = 0.f, tail_s = 0.f, tail_t = 0.f;
  bool with_tail = false, tail_grad = false;
  if (p.norm == RELAX_AMD_OPD_NORM_NORM) {
    shift_s = ls;
    shift_t = lt;
  } else if (p.norm == RELAX_AMD_OPD_NORM_TAIL) {
    // tail bin log(1 - sum p) with the log-sum-exp clamped to <= -1e-7; the union path's mask cuts it off again
    tail_s = logf(-expm1f(fminf(ls, -1e-7f)));
    tail_t = logf(-expm1f(fminf(lt, -1e-7f)));
    with_tail = !has_mask;
    tail_grad = ls <= -1e-7f;
  }
  const float log_1ma = logf(1.f - p.alpha), log_a = logf(p.alpha);
  float acc = 0.f, dsum = 0.f;
  for (int k = lane; k < k_ids; k += kWave) {
    if (has_mask && !valid(k)) continue;
    float term, dterm;
    opd_entry(sv[k] - shift_s, tv[k] - shift_t, p.alpha, log_1ma, log_a, term, dterm);
    acc += term;
    dsum += dterm;
  }
  acc = wave_sum(acc);
  float d_tail = 0.f;
  if (with_tail) {
    float term;
    opd_entry(tail_s, tail_t, p.alpha, log_1ma, log_a, term, d_tail);
    acc += term;
  }
  if (!BWD) return acc;
  dsum = wave_sum(dsum);
  for (int k = lane; k < k_ids; k += kWave) {
    float dk = 0.f;
    bool nonzero = false;
    if (!has_mask || valid(k)) {
      float term, dterm;
      opd_entry(sv[k] - shift_s, tv[k] - shift_t, p.alpha, log_1ma, log_a, term, dterm);
      dk = dterm;
      if (p.norm == RELAX_AMD_OPD_NORM_NORM) dk -= expf(sv[k] - ls) * dsum;
      if (with_tail && tail_grad) dk -= d_tail * expf(sv[k] - tail_s);
      nonzero = !(p.has_clamp && !(load_s(k) >= p.clamp));
    }
    store_d(k, dk, nonzero);
  }
  return acc;
}

// Host-side check of the optional top-K distillation block of the fused actor step; NULL when it is consistent.
inline const char* topk_distill_args_error(const relax_amd_policy_loss_args& a) {
  if (!a.topk_ids) return nullptr;
  if (!a.extra_coef_log_prob) return "topk_ids needs extra_coef_log_prob (the signal's weights)";
  if (a.distill_teacher_log_prob) return "topk_ids and distill_teacher_log_prob are alternatives";
  if (!a.topk_teacher_log_prob || !a.topk_kl || !a.topk_grad) return "topk_ids needs topk_teacher_log_prob, topk_kl and topk_grad";
  if (a.topk_k < 1 || a.topk_k > RELAX_AMD_FUSED_TOPK_MAX) return "topk_k must be in 1..RELAX_AMD_FUSED_TOPK_MAX";
  if ((a.topk_kl_mode != RELAX_AMD_OPD_JSD && a.topk_kl_mode != RELAX_AMD_OPD_LOW_VAR) ||
      a.topk_norm_mode < RELAX_AMD_OPD_NORM_TAIL || a.topk_norm_mode > RELAX_AMD_OPD_NORM_TRUNC ||
      !(a.topk_jsd_alpha >= 0.f && a.topk_jsd_alpha <= 1.f))
    return "unknown topk_kl_mode / topk_norm_mode, or topk_jsd_alpha outside [0, 1]";
  return nullptr;
}

// What a lane of the first wave requests ahead of time for the top-K distillation signal of a token: the row's logits
// at its ids (entries lane, lane + 64, ...) and the teacher's log-probs there.  Nothing here depends on the row's
// log-sum-exp, so the two dependent gathers (ids, then logits) are requested before the workgroup merges its scan
// (the merge's barrier waits for them: they overlap the other waves' way to that barrier, not the merge itself).
constexpr int kTopkPerLane = RELAX_AMD_FUSED_TOPK_MAX / kWave;
struct TopkGather {
  float x[kTopkPerLane];  // the gathered logit; -inf for a sentinel id, 0 for an id outside the vocabulary
  float t[kTopkPerLane];
  bool real[kTopkPerLane];  // the id is not a sentinel (its log-prob carries the row's log-sum-exp)
};

template <typename T>
__device__ __forceinline__ TopkGather topk_gather(const relax_amd_policy_loss_args& a, const T* x, int64_t vocab,
                                                  int64_t tok, int lane) {
  TopkGather g;
  const int kmax = a.topk_k;
  const int64_t* ids = a.topk_ids + tok * kmax;
  const float* teacher = a.topk_teacher_log_prob + tok * kmax;
#pragma unroll
  for (int i = 0; i < kTopkPerLane; ++i) {
    const int k = lane + i * kWave;
    g.x[i] = g.t[i] = 0.f;
    g.real[i] = false;
    if (k < kmax) {
      const int64_t id = ids[k];
      g.t[i] = teacher[k];
      g.real[i] = id >= 0;
      // a sentinel yields log-prob -inf; outside the vocabulary slice the reference gathers a zero logit
      g.x[i] = id < 0 ? -INFINITY : (id >= vocab ? 0.f : Row<T>::load1(x + id));
    }
  }
  return g;
}

// topk_gather() without the logits (x stays 0): the teacher's log-probs and which ids are sentinels, both contiguous
// reads, for a caller that receives the gathered logits from elsewhere (the one-shot actor step shares the scattered
// gather between the workgroups of a row).
__device__ __forceinline__ TopkGather topk_gather_meta(const relax_amd_policy_loss_args& a, int64_t tok, int lane) {
  TopkGather g;
  const int kmax = a.topk_k;
  const int64_t* ids = a.topk_ids + tok * kmax;
  const float* teacher = a.topk_teacher_log_prob + tok * kmax;
#pragma unroll
  for (int i = 0; i < kTopkPerLane; ++i) {
    const int k = lane + i * kWave;
    g.x[i] = g.t[i] = 0.f;
    g.real[i] = false;
    if (k < kmax) {
      g.t[i] = teacher[k];
      g.real[i] = ids[k] >= 0;
    }
  }
  return g;
}
// the logit topk_gather() puts in x for entry k of token `tok`
template <typename T>
__device__ __forceinline__ float topk_gather_one(const relax_amd_policy_loss_args& a, const T* x, int64_t vocab,
                                                 int64_t id) {
  return id < 0 ? -INFINITY : (id >= vocab ? 0.f : Row<T>::load1(x + id));
}

// Token `tok`'s entry count and union-mask length for the signal (the whole list / no mask without the arrays): two
// more scalars that can be on their way before the row's log-sum-exp is known.
struct TopkRowShape {
  int width, nvalid;
};
__device__ __forceinline__ TopkRowShape topk_row_shape(const relax_amd_policy_loss_args& a, int64_t tok) {
  return {a.topk_width ? a.topk_width[tok] : a.topk_k, a.topk_valid ? a.topk_valid[tok] : -1};
}

// The top-K distillation signal of one token inside the fused actor step, by the workgroup's first wave once the row's
// log-sum-exp is known: log-probs at the token's K ids (as topk_logprob_fwd_kernel forms them), the per-token KL,
// clips and weight, topk_kl / topk_grad written.  `g` = this lane's topk_gather(), `shape` = topk_row_shape() of the
// token, `weight` = the signal's weight in the loss, `old` = the token's old log-prob (the current one when there is
// none).  Returns, in every lane, the sum of d loss / d log p[id_k] over the non-sentinel ids: what the row's softmax
// is multiplied by, next to the policy terms' own coefficient.  `stage` = kTopkStageFloats floats of LDS.  `emit`:
// whether this caller writes topk_kl / topk_grad (one of several workgroups that evaluate the same token does).
constexpr int kTopkStageFloats = 4 * RELAX_AMD_FUSED_TOPK_MAX;

__device__ __forceinline__ float topk_distill_row(const relax_amd_policy_loss_args& a, const TopkGather& g,
                                                  const TopkRowShape& shape, int64_t tok, float lse, float inv_t,
                                                  float lp, float old, float weight, int lane, float* stage,
                                                  bool emit = true) {
  const int kmax = a.topk_k;
  const int width = shape.width < 0 ? 0 : (shape.width > kmax ? kmax : shape.width);
  const int nvalid = shape.nvalid;
  const OpdParams p{a.topk_kl_mode, a.topk_norm_mode, a.topk_jsd_alpha, a.topk_has_clamp, a.topk_min_clamp};
  float* sv = stage;
  float* tv = stage + RELAX_AMD_FUSED_TOPK_MAX;
  float* raw_s = stage + 2 * RELAX_AMD_FUSED_TOPK_MAX;  // the student log-probs before clamp and mask
  float* raw_t = stage + 3 * RELAX_AMD_FUSED_TOPK_MAX;
#pragma unroll
  for (int i = 0; i < kTopkPerLane; ++i) {
    const int k = lane + i * kWave;
    if (k < kmax) {
      raw_s[k] = fmaf(g.x[i], inv_t, -lse);
      raw_t[k] = g.t[i];
    }
  }
  // the derivatives land in sv[] (store_d is the last use of an entry's staged values)
  const float kl = opd_kl_row<true>(
      width, nvalid >= 0, p, lane, sv, tv, [&](int k) { return raw_s[k]; }, [&](int k) { return raw_t[k]; },
      [&](int k) { return k < nvalid; }, [&](int k, float dk, bool nonzero) { sv[k] = nonzero ? dk : 0.f; });
  float pass = 1.f;
  if (a.distill_token_clip == a.distill_token_clip && kl > a.distill_token_clip) pass = 0.f;
  if (a.distill_is_clip == a.distill_is_clip) pass *= fminf(expf(lp - old), a.distill_is_clip);
  const float f = weight * pass;
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < kTopkPerLane; ++i) {
    const int k = lane + i * kWave;
    if (k < kmax) {
      float d = 0.f;
      if (k < width && sv[k] != 0.f) {  // entries without gradient stay exact zeros whatever the weight holds
        d = f * sv[k];
        if (g.real[i] && d != 0.f) total += d;
      }
      if (emit) a.topk_grad[tok * kmax + k] = d;
    }
  }
  if (lane == 0 && emit) a.topk_kl[tok] = kl;
  return wave_sum(total);
}

}  // namespace relax_amd
