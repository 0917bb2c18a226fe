// Per-token policy loss + KL penalty + masked per-sample aggregation + gradient coefficients, in two launches.
//
// Launch 1: one workgroup per sample (a response in the packed "thd" layout, delimited by cu_resp).  The workgroup
// walks its tokens up to three times over KB-sized fp32 side vectors (never over logits):
//   pass A (GSPO / OPSM only)  sequence KL  k_i = sum((old-lp)*m) / max(sum m, 1)        ppo_utils.py:183-209, 142-180
//   pass B                     per-token loss terms, masked sums of every metric, and the token-local part of
//                              d loss / d lp;  for GSPO also G_i = sum_t w_t * A_t * r_i * [unclipped]
//   pass C (GSPO only)         adds the sequence-coupled gradient  -G_i * m_t / max(sum m, 1)
// Per-sample sums are divided by the caller's per-sample denominators, exactly the structure of
// get_sum_of_sample_mean / sum_of_token (relax/backends/megatron/cp_utils.py:144-162).
// Launch 2: one workgroup adds the per-sample partials in sample order and assembles
//   loss = pg_loss - entropy_coef * entropy_loss + kl_coef * kl_loss                        loss.py:1084-1100
// All reductions use a fixed combination order, so results are bit-identical run to run.
//
// Gradient conventions reproduced from autograd over the reference's torch ops:
//   PPO-clip   d/dlp = -A*r when r is inside [1-eps_lo, 1+eps_hi] or the unclipped branch is strictly larger, else 0
//   dual clip  A<0 and -c*A < clipped loss: 0; tie: half
//   CISPO      -coef*A (coef, A detached);  RLOO  -A;  SAPO  -A*4*s*(1-s)*r  (s = sigmoid(tau*(r-1)))
//   k1: 1   k2: d   k3 / low_var: 1-exp(-d)  (low_var: 0 outside the [-10,10] clamp)
//   unbiased KL multiplies by ratio = exp(lp-old) and adds ratio*kl (the ratio is not detached, loss.py:1091)
#include "device_utils.h"
#include "loss_math.h"
#include "relax_amd.h"

namespace relax_amd {

constexpr int kLossThreads = 512;

__global__ __launch_bounds__(kLossThreads) void policy_loss_sample_kernel(relax_amd_policy_loss_args a) {
  __shared__ float red[kLossThreads / kWave];
  const int64_t i = blockIdx.x;
  const int64_t beg = a.cu_resp[i], end = a.cu_resp[i + 1];
  const bool gspo = a.loss_kind == RELAX_AMD_LOSS_GSPO;
  const float den = a.sample_denom ? a.sample_denom[i] : 1.0f;
  const float pg_den = a.pg_sample_denom ? a.pg_sample_denom[i] : den;

  float seq_kl = 0.f, seq_cnt = 1.f;
  if (gspo || a.use_opsm) {
    float sd = 0.f, sm = 0.f;
    for (int64_t t = beg + threadIdx.x; t < end; t += kLossThreads) {
      const float lp = a.log_prob[t];
      const float old = a.old_log_prob ? a.old_log_prob[t] : lp;
      const float m = a.loss_mask[t];
      sd += (old - lp) * m;
      sm += m;
    }
    sd = block_sum<kLossThreads>(sd, red);
    sm = block_sum<kLossThreads>(sm, red);
    seq_cnt = fmaxf(sm, 1.0f);
    seq_kl = sd / seq_cnt;
  }

  float acc[RELAX_AMD_NUM_METRICS];
#pragma unroll
  for (int k = 0; k < RELAX_AMD_NUM_METRICS; ++k) acc[k] = 0.f;
  float g_seq = 0.f;  // GSPO: sum_t w_t * d pg_t / d kl_i

  for (int64_t t = beg + threadIdx.x; t < end; t += kLossThreads) {
    const TokenInputs in = load_token_inputs(a, t);
    TokenResult tr = token_terms(a, in, a.log_prob[t], a.entropy ? a.entropy[t] : 0.f, gspo, seq_kl, den, pg_den);
#pragma unroll
    for (int k = 0; k < RELAX_AMD_NUM_METRICS; ++k) acc[k] += tr.metric[k];
    g_seq += tr.g_seq;
    if (a.pg_loss_tok) a.pg_loss_tok[t] = tr.pg;
    if (a.clipfrac_tok) a.clipfrac_tok[t] = tr.clipfrac;
    if (a.ppo_kl_tok) a.ppo_kl_tok[t] = tr.ppo_kl;
    if (a.kl_tok && a.kl_kind != RELAX_AMD_KL_NONE) a.kl_tok[t] = tr.kl;
    a.coef_log_prob[t] = tr.coef_lp;
    if (a.coef_entropy) a.coef_entropy[t] = tr.coef_ent;
  }

#pragma unroll
  for (int k = 0; k < RELAX_AMD_NUM_METRICS; ++k) acc[k] = block_sum<kLossThreads>(acc[k], red);
  if (gspo) {
    g_seq = block_sum<kLossThreads>(g_seq, red);
    // d kl_i / d lp_t = -m_t / max(sum m, 1)
    for (int64_t t = beg + threadIdx.x; t < end; t += kLossThreads)
      a.coef_log_prob[t] += g_seq * (-a.loss_mask[t] / seq_cnt);
  }
  if (threadIdx.x == 0) {
    float* out = a.sample_partials + i * RELAX_AMD_NUM_METRICS;
    out[RELAX_AMD_M_LOSS] = 0.f;
    out[RELAX_AMD_M_PG_LOSS] = acc[RELAX_AMD_M_PG_LOSS] / pg_den;
    out[RELAX_AMD_M_MASK_SUM] = acc[RELAX_AMD_M_MASK_SUM];
    // opsm_clipfrac: dropped-token count over max(sum m, 1) of the sample (ppo_utils.py:175)
    out[RELAX_AMD_M_OPSM_CLIPFRAC] = acc[RELAX_AMD_M_OPSM_CLIPFRAC] / fmaxf(acc[RELAX_AMD_M_MASK_SUM], 1.0f);
#pragma unroll
    for (int k = RELAX_AMD_M_ENTROPY; k <= RELAX_AMD_M_MISMATCH_K3; ++k) out[k] = acc[k] / den;
  }
}

// Sums the per-sample partial metrics in sample order (one lane per metric, each a plain sequence of fp32 additions,
// so the result does not depend on how many samples a launch stages at a time).  The partials are staged through LDS
// by the whole workgroup, 512 samples at a time: a lane adding straight from global memory waits out one memory
// latency per sample (74 us for 512 samples).
constexpr int kFinishThreads = 256;
constexpr int kFinishStage = 512;  // samples per staging round (32 KB)

__global__ __launch_bounds__(kFinishThreads) void policy_loss_finish_kernel(const float* __restrict__ partials,
                                                                           int64_t n_samples, float entropy_coef,
                                                                           float kl_coef, int has_kl,
                                                                           float* __restrict__ metrics) {
  __shared__ float stage[kFinishStage * RELAX_AMD_NUM_METRICS];
  const int k = threadIdx.x;
  float total = 0.f;
  for (int64_t base = 0; base < n_samples; base += kFinishStage) {
    const int count = int(n_samples - base < kFinishStage ? n_samples - base : kFinishStage);
    for (int e = k; e < count * RELAX_AMD_NUM_METRICS; e += kFinishThreads)
      stage[e] = partials[base * RELAX_AMD_NUM_METRICS + e];
    __syncthreads();
    if (k < RELAX_AMD_NUM_METRICS)
      for (int i = 0; i < count; ++i) total += stage[i * RELAX_AMD_NUM_METRICS + k];
    __syncthreads();
  }
  if (k >= kWave) return;
  const float pg = lane_value<RELAX_AMD_M_PG_LOSS>(total);
  const float ent = lane_value<RELAX_AMD_M_ENTROPY>(total);
  const float kl = lane_value<RELAX_AMD_M_KL_LOSS>(total);
  if (k == RELAX_AMD_M_LOSS) {
    total = pg - entropy_coef * ent;
    if (has_kl) total = total + kl_coef * kl;
  }
  if (k < RELAX_AMD_NUM_METRICS) metrics[k] = total;
}

__global__ __launch_bounds__(256) void segment_sum_kernel(const float* __restrict__ values,
                                                          const float* __restrict__ mask,
                                                          const int64_t* __restrict__ cu, double* __restrict__ out) {
  __shared__ double red[256 / kWave];
  const int64_t i = blockIdx.x;
  double s = 0.0;
  for (int64_t t = cu[i] + threadIdx.x; t < cu[i + 1]; t += 256)
    s += values ? double(values[t] * mask[t]) : double(mask[t]);
  s = block_sum<256>(s, red);
  if (threadIdx.x == 0) out[i] = s;
}

__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* __restrict__ p, int64_t n, int32_t v) {
  for (int64_t i = blockIdx.x * 256LL + threadIdx.x; i < n; i += int64_t(gridDim.x) * 256) p[i] = v;
}

__global__ __launch_bounds__(256) void row_maps_kernel(const int64_t* __restrict__ row_begin,
                                                       const int64_t* __restrict__ cu, int64_t n_rows,
                                                       int32_t* __restrict__ row_ids, int32_t* __restrict__ sample_ids,
                                                       int32_t* __restrict__ token_of_row) {
  const int64_t i = blockIdx.x;
  const int64_t beg = cu[i], len = cu[i + 1] - cu[i], r0 = row_begin[i];
  for (int64_t j = threadIdx.x; j < len; j += 256) {
    const int64_t row = r0 + j;
    row_ids[beg + j] = int32_t(row);
    if (sample_ids) sample_ids[beg + j] = int32_t(i);
    if (token_of_row && row >= 0 && row < n_rows) token_of_row[row] = int32_t(beg + j);
  }
}

// Target ids of the packed response tokens, gathered from the packed token ids: sample i's j-th target sits at
// src_begin[i] + j of `tokens`, or is 0 when that position is past src_end[i] (the SFT layout's final pad).
__global__ __launch_bounds__(256) void gather_targets_kernel(const int64_t* __restrict__ tokens,
                                                             const int64_t* __restrict__ src_begin,
                                                             const int64_t* __restrict__ src_end,
                                                             const int64_t* __restrict__ cu,
                                                             int64_t* __restrict__ targets) {
  const int64_t i = blockIdx.x;
  const int64_t beg = cu[i], len = cu[i + 1] - cu[i], s0 = src_begin[i], s1 = src_end[i];
  for (int64_t j = threadIdx.x; j < len; j += 256) targets[beg + j] = (s0 + j < s1) ? tokens[s0 + j] : 0;
}

}  // namespace relax_amd

using namespace relax_amd;

extern "C" int relax_amd_gather_targets(const int64_t* tokens, const int64_t* src_begin, const int64_t* src_end,
                                        const int64_t* cu_resp, int64_t n_samples, int64_t* targets, void* stream) {
  if (n_samples < 0 || n_samples > 2147483647LL) {
    set_error("gather_targets: bad n_samples=%lld", (long long)n_samples);
    return RELAX_AMD_EINVAL;
  }
  if (n_samples == 0) return RELAX_AMD_OK;
  if (!tokens || !src_begin || !src_end || !cu_resp || !targets) {
    set_error("gather_targets: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipLaunchKernelGGL(gather_targets_kernel, dim3(static_cast<unsigned>(n_samples)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), tokens, src_begin, src_end, cu_resp, targets);
  return check_launch("gather_targets");
}

extern "C" int relax_amd_policy_loss(const relax_amd_policy_loss_args* a, void* stream) {
  if (!a) {
    set_error("policy_loss: args is NULL");
    return RELAX_AMD_EINVAL;
  }
  if (policy_loss_args_size_error(a)) {
    set_error("policy_loss: %s", policy_loss_args_size_error(a));
    return RELAX_AMD_EINVAL;
  }
  if (a->n_samples < 0 || a->n_tokens < 0 || a->n_samples > 2147483647LL) {
    set_error("policy_loss: bad sizes n_samples=%lld n_tokens=%lld", (long long)a->n_samples, (long long)a->n_tokens);
    return RELAX_AMD_EINVAL;
  }
  if (!a->metrics || !a->sample_partials || !a->cu_resp) {
    set_error("policy_loss: metrics, sample_partials and cu_resp must not be NULL");
    return RELAX_AMD_EINVAL;
  }
  if (a->n_tokens > 0 && (!a->log_prob || !a->advantages || !a->loss_mask || !a->coef_log_prob)) {
    set_error("policy_loss: log_prob, advantages, loss_mask and coef_log_prob must not be NULL");
    return RELAX_AMD_EINVAL;
  }
  if (const char* why = distill_args_error(*a)) {
    set_error("policy_loss: %s", why);
    return RELAX_AMD_EINVAL;
  }
  if (a->loss_kind < RELAX_AMD_LOSS_PPO || a->loss_kind > RELAX_AMD_LOSS_SAPO) {
    set_error("policy_loss: unknown loss_kind %d", a->loss_kind);
    return RELAX_AMD_EINVAL;
  }
  if (a->kl_kind < RELAX_AMD_KL_NONE || a->kl_kind > RELAX_AMD_KL_LOW_VAR) {
    set_error("policy_loss: unknown kl_kind %d", a->kl_kind);
    return RELAX_AMD_EINVAL;
  }
  if (a->kl_kind != RELAX_AMD_KL_NONE && a->n_tokens > 0 && !a->ref_log_prob) {
    set_error("policy_loss: ref_log_prob is required when kl_kind != NONE");
    return RELAX_AMD_EINVAL;
  }
  if (a->eps_clip_c > 0.f && !(a->eps_clip_c > 1.0f)) {
    set_error("policy_loss: eps_clip_c must be > 1.0 (got %f)", a->eps_clip_c);
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (a->n_samples > 0) {
    hipLaunchKernelGGL(policy_loss_sample_kernel, dim3(static_cast<unsigned>(a->n_samples)), dim3(kLossThreads), 0, s,
                       *a);
    int rc = check_launch("policy_loss_sample");
    if (rc) return rc;
  }
  hipLaunchKernelGGL(policy_loss_finish_kernel, dim3(1), dim3(kFinishThreads), 0, s, a->sample_partials, a->n_samples,
                     a->entropy_coef, a->kl_coef, int(a->kl_kind != RELAX_AMD_KL_NONE), a->metrics);
  return check_launch("policy_loss_finish");
}

extern "C" int relax_amd_segment_sum(const float* values, const float* mask, const int64_t* cu_resp, int64_t n_samples,
                                     double* out, void* stream) {
  if (n_samples < 0 || n_samples > 2147483647LL) {
    set_error("segment_sum: bad n_samples %lld", (long long)n_samples);
    return RELAX_AMD_EINVAL;
  }
  if (n_samples == 0) return RELAX_AMD_OK;
  if (!mask || !cu_resp || !out) {
    set_error("segment_sum: mask, cu_resp and out must not be NULL");
    return RELAX_AMD_EINVAL;
  }
  hipLaunchKernelGGL(segment_sum_kernel, dim3(static_cast<unsigned>(n_samples)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), values, mask, cu_resp, out);
  return check_launch("segment_sum");
}

extern "C" int relax_amd_build_row_maps(const int64_t* row_begin, const int64_t* cu_resp, int64_t n_samples,
                                        int64_t n_tokens, int64_t n_rows, int32_t* row_ids, int32_t* sample_ids,
                                        int32_t* token_of_row, void* stream) {
  if (n_samples < 0 || n_tokens < 0 || n_rows < 0 || n_rows > 2147483647LL || n_tokens > 2147483647LL ||
      n_samples > 2147483647LL) {
    set_error("build_row_maps: bad sizes");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (token_of_row && n_rows > 0) {
    const unsigned blocks = static_cast<unsigned>((n_rows + 255) / 256 > 4096 ? 4096 : (n_rows + 255) / 256);
    hipLaunchKernelGGL(fill_i32_kernel, dim3(blocks), dim3(256), 0, s, token_of_row, n_rows, int32_t(-1));
    int rc = check_launch("fill_i32");
    if (rc) return rc;
  }
  if (n_samples == 0 || n_tokens == 0) return RELAX_AMD_OK;
  if (!row_begin || !cu_resp || !row_ids) {
    set_error("build_row_maps: row_begin, cu_resp and row_ids must not be NULL");
    return RELAX_AMD_EINVAL;
  }
  hipLaunchKernelGGL(row_maps_kernel, dim3(static_cast<unsigned>(n_samples)), dim3(256), 0, s, row_begin, cu_resp,
                     n_rows, row_ids, sample_ids, token_of_row);
  return check_launch("row_maps");
}
