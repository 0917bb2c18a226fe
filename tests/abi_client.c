/* A C program that uses the library the way a non-Python host would: plain pointers from hipMalloc, the declarations
 * of include/relax_amd.h, no PyTorch.  It runs the log-prob / entropy forward and its dlogits backward on the
 * three-row case of the reference's tests/utils/training/test_ppo_logprob_entropy.py:174-263 (logits
 * [[1,2,3,4],[4,1,0.5,2],[-1,3,2,0]], tokens [3,0,1], weights [0.25,-0.5,1.5] / [0.55,-0.2,1.8]) and the reverse KL
 * of two rows, and compares with the closed forms evaluated here in double precision; then the one-read log-prob +
 * top-K entry point on the same rows (k = 2) and the group-normalised rewards of the reference's GRPO literal
 * (tests/utils/training/test_rloo_advantages.py:160-172: rewards [0,1,0,1] in one group -> (r - 0.5) / (std + 1e-6)
 * with the sample standard deviation) and its leave-one-out brute force; then the fused actor step with the top-K
 * distillation term (relax_amd_actor_step_fused + relax_amd_sparse_row_add + relax_amd_policy_loss) against its closed
 * form.  Exit status 0 = all good. */
#include <hip/hip_runtime_api.h>
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include "relax_amd.h"

#define CHECK_HIP(x)                                                                \
  do {                                                                              \
    hipError_t e_ = (x);                                                            \
    if (e_ != hipSuccess) {                                                         \
      fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));                       \
      return 2;                                                                     \
    }                                                                               \
  } while (0)
#define CHECK_LIB(x)                                                                \
  do {                                                                              \
    int rc_ = (x);                                                                  \
    if (rc_ != RELAX_AMD_OK) {                                                      \
      fprintf(stderr, "%s -> %d: %s\n", #x, rc_, relax_amd_last_error());           \
      return 3;                                                                     \
    }                                                                               \
  } while (0)

enum { N = 3, V = 4 };

static int close_enough(const char* what, int i, double got, double want, double tol) {
  if (fabs(got - want) <= tol) return 1;
  fprintf(stderr, "%s[%d]: got %.9g, want %.9g\n", what, i, got, want);
  return 0;
}

static void* to_device(const void* host, size_t bytes) {
  void* p = NULL;
  if (hipMalloc(&p, bytes) != hipSuccess) return NULL;
  if (host && hipMemcpy(p, host, bytes, hipMemcpyHostToDevice) != hipSuccess) return NULL;
  return p;
}

int main(void) {
  const float logits[N][V] = {{1, 2, 3, 4}, {4, 1, 0.5f, 2}, {-1, 3, 2, 0}};
  const float teacher[N][V] = {{0.5f, 2, 2.5f, 4}, {4, 1, 0.5f, 2}, {0, 0, 0, 0}};
  const int64_t tokens[N] = {3, 0, 1};
  const float w_lp[N] = {0.25f, -0.5f, 1.5f}, w_ent[N] = {0.55f, -0.2f, 1.8f};
  int count = 0;
  CHECK_HIP(hipGetDeviceCount(&count));
  if (count < 1) {
    fprintf(stderr, "no GPU\n");
    return 2;
  }
  CHECK_HIP(hipSetDevice(0));
  hipStream_t stream;
  CHECK_HIP(hipStreamCreate(&stream));
  void* d_logits = to_device(logits, sizeof logits);
  void* d_teacher = to_device(teacher, sizeof teacher);
  void* d_tokens = to_device(tokens, sizeof tokens);
  void* d_wlp = to_device(w_lp, sizeof w_lp);
  void* d_went = to_device(w_ent, sizeof w_ent);
  float *d_lp = to_device(NULL, N * sizeof(float)), *d_ent = to_device(NULL, N * sizeof(float));
  float *d_lse = to_device(NULL, N * sizeof(float)), *d_spx = to_device(NULL, N * sizeof(float));
  float *d_kl = to_device(NULL, N * sizeof(float)), *d_ls = to_device(NULL, N * sizeof(float));
  float* d_lt = to_device(NULL, N * sizeof(float));
  void* d_grad = to_device(NULL, sizeof logits);
  if (!d_logits || !d_teacher || !d_tokens || !d_wlp || !d_went || !d_lp || !d_ent || !d_lse || !d_spx || !d_kl ||
      !d_ls || !d_lt || !d_grad) {
    fprintf(stderr, "device allocation failed\n");
    return 2;
  }

  CHECK_LIB(relax_amd_logprob_entropy_fwd(d_logits, RELAX_AMD_F32, N, V, V, NULL, (const int64_t*)d_tokens, 1.0f, d_lp,
                                          d_ent, d_lse, d_spx, stream));
  CHECK_LIB(relax_amd_logprob_entropy_bwd(d_logits, RELAX_AMD_F32, N, V, V, NULL, (const int64_t*)d_tokens, d_lse,
                                          d_spx, (const float*)d_wlp, (const float*)d_went, 1.0f, NULL, 1.0f, d_grad, V,
                                          stream));
  CHECK_LIB(relax_amd_reverse_kl_fwd(d_logits, d_teacher, RELAX_AMD_F32, N, V, V, d_kl, d_ls, d_lt, stream));
  CHECK_HIP(hipStreamSynchronize(stream));

  float lp[N], ent[N], kl[N], grad[N][V];
  CHECK_HIP(hipMemcpy(lp, d_lp, sizeof lp, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(ent, d_ent, sizeof ent, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(kl, d_kl, sizeof kl, hipMemcpyDeviceToHost));
  CHECK_HIP(hipMemcpy(grad, d_grad, sizeof grad, hipMemcpyDeviceToHost));

  int ok = 1;
  for (int i = 0; i < N; ++i) {
    double z = 0, zt = 0, px = 0;
    for (int v = 0; v < V; ++v) {
      z += exp((double)logits[i][v]);
      zt += exp((double)teacher[i][v]);
    }
    const double lse = log(z), lset = log(zt);
    double want_kl = 0;
    for (int v = 0; v < V; ++v) {
      const double p = exp(logits[i][v] - lse);
      px += p * logits[i][v];
      want_kl += p * ((logits[i][v] - lse) - (teacher[i][v] - lset));
    }
    ok &= close_enough("log_prob", i, lp[i], logits[i][tokens[i]] - lse, 2e-6);
    ok &= close_enough("entropy", i, ent[i], lse - px, 2e-6);
    ok &= close_enough("reverse_kl", i, kl[i], want_kl, 2e-6);
    for (int v = 0; v < V; ++v) {
      const double p = exp(logits[i][v] - lse);
      const double want = w_lp[i] * ((v == tokens[i]) - p) + w_ent[i] * p * (px - logits[i][v]);
      ok &= close_enough("dlogits", i * V + v, grad[i][v], want, 2e-6);
    }
  }
  /* log-probs + entropy + the two largest logits of every row from one entry point */
  {
    enum { K = 2 };
    float *d_lp2 = to_device(NULL, N * sizeof(float)), *d_vals = to_device(NULL, N * K * sizeof(float));
    int64_t* d_idx = to_device(NULL, N * K * sizeof(int64_t));
    uint8_t* d_flags = to_device(NULL, N);
    if (!d_lp2 || !d_vals || !d_idx || !d_flags) return 2;
    CHECK_LIB(relax_amd_logprob_entropy_topk_fwd(d_logits, RELAX_AMD_F32, N, V, V, NULL, (const int64_t*)d_tokens, 1.0f,
                                                 K, d_lp2, NULL, NULL, NULL, d_vals, d_idx, d_flags, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    float lp2[N], vals[N][K];
    int64_t idx[N][K];
    CHECK_HIP(hipMemcpy(lp2, d_lp2, sizeof lp2, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(vals, d_vals, sizeof vals, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(idx, d_idx, sizeof idx, hipMemcpyDeviceToHost));
    const int64_t want_idx[N][K] = {{3, 2}, {0, 3}, {1, 2}};
    for (int i = 0; i < N; ++i) {
      ok &= close_enough("topk log_prob", i, lp2[i], lp[i], 0.0);
      for (int k = 0; k < K; ++k) {
        ok &= close_enough("topk index", i * K + k, (double)idx[i][k], (double)want_idx[i][k], 0.0);
        ok &= close_enough("topk value", i * K + k, vals[i][k], logits[i][want_idx[i][k]], 0.0);
      }
    }
  }
  /* group-normalised rewards: mean / sample-std normalisation and leave-one-out baselines of one group of four */
  {
    enum { G = 4 };
    const float rewards[G] = {0, 1, 0, 1};
    const int32_t group[G] = {0, 0, 0, 0};
    void* d_r = to_device(rewards, sizeof rewards);
    void* d_g = to_device(group, sizeof group);
    float* d_out = to_device(NULL, sizeof rewards);
    int32_t* d_cnt = to_device(NULL, sizeof group);
    if (!d_r || !d_g || !d_out || !d_cnt) return 2;
    float out[G];
    int32_t cnt[G];
    CHECK_LIB(relax_amd_group_rewards(d_r, RELAX_AMD_F32, (const int32_t*)d_g, G, RELAX_AMD_GROUP_CENTER_STD, d_out, d_cnt,
                                      stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    CHECK_HIP(hipMemcpy(out, d_out, sizeof out, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(cnt, d_cnt, sizeof cnt, hipMemcpyDeviceToHost));
    const double sd = sqrt(4 * 0.25 / 3.0);  /* sample standard deviation of {0,1,0,1} */
    for (int i = 0; i < G; ++i) {
      ok &= close_enough("grpo reward", i, out[i], (rewards[i] - 0.5) / (sd + 1e-6), 1e-6);
      ok &= close_enough("group size", i, cnt[i], G, 0.0);
    }
    CHECK_LIB(relax_amd_group_rewards(d_r, RELAX_AMD_F32, (const int32_t*)d_g, G, RELAX_AMD_GROUP_RLOO, d_out, d_cnt,
                                      stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    CHECK_HIP(hipMemcpy(out, d_out, sizeof out, hipMemcpyDeviceToHost));
    for (int i = 0; i < G; ++i) {
      double others = 0;
      for (int j = 0; j < G; ++j)
        if (j != i) others += rewards[j];
      ok &= close_enough("rloo reward", i, out[i], rewards[i] - others / (G - 1), 1e-6);
    }
  }
  /* the fused actor step with the top-K distillation term, from C: PPO at ratio 1 (no old log-probs), token-mean over
   * one sample of three tokens, plus 0.5 * mean_t KL_t with KL_t = sum_k p_k (log p_k - teacher_k) over two given ids
   * per row (reverse KL, entries used as they are); then the K one-hot parts; against the closed forms:
   *   dlogits[t, v] = -(A_t / 3) (1[v = token_t] - p_v) + sum_k w d_k (1[v = id_k] - p_v),  d_k = p_k (log p_k - teacher_k + 1) */
  {
    enum { K = 2 };
    const float adv[N] = {1.0f, -2.0f, 0.5f}, ones[N] = {1, 1, 1}, denom[1] = {3.0f};
    const int64_t cu[2] = {0, N}, ids[N][K] = {{3, 1}, {0, 2}, {1, 3}};
    const int32_t sample_ids[N] = {0, 0, 0};
    const float teacher_lp[N][K] = {{-0.5f, -2.0f}, {-0.3f, -3.0f}, {-1.0f, -1.5f}};
    const float w = 0.5f / 3.0f, weight[N] = {w, w, w};
    void *d_adv = to_device(adv, sizeof adv), *d_mask = to_device(ones, sizeof ones), *d_den = to_device(denom, sizeof denom);
    void *d_cu = to_device(cu, sizeof cu), *d_ids = to_device(ids, sizeof ids), *d_sid = to_device(sample_ids, sizeof sample_ids);
    void *d_tlp = to_device(teacher_lp, sizeof teacher_lp), *d_w = to_device(weight, sizeof weight);
    float *d_coef = to_device(NULL, N * sizeof(float)), *d_part = to_device(NULL, RELAX_AMD_NUM_METRICS * sizeof(float));
    float *d_met = to_device(NULL, RELAX_AMD_NUM_METRICS * sizeof(float)), *d_tkl = to_device(NULL, N * sizeof(float));
    float* d_tgrad = to_device(NULL, N * K * sizeof(float));
    float *d_lp3 = to_device(NULL, N * sizeof(float)), *d_ent3 = to_device(NULL, N * sizeof(float));
    if (!d_adv || !d_mask || !d_den || !d_cu || !d_ids || !d_sid || !d_tlp || !d_w || !d_coef || !d_part || !d_met ||
        !d_tkl || !d_tgrad || !d_lp3 || !d_ent3)
      return 2;
    relax_amd_policy_loss_args a = {0};
    a.struct_size = sizeof(a);
    a.advantages = d_adv;
    a.loss_mask = d_mask;
    a.cu_resp = d_cu;
    a.sample_denom = d_den;
    a.n_samples = 1;
    a.n_tokens = N;
    a.loss_kind = RELAX_AMD_LOSS_PPO;
    a.kl_kind = RELAX_AMD_KL_NONE;
    a.eps_clip = a.eps_clip_high = 0.2f;
    a.eps_clip_c = -1.0f;
    a.tis_hi = 2.0f;
    a.coef_log_prob = d_coef;
    a.sample_partials = d_part;
    a.metrics = d_met;
    a.extra_coef_log_prob = d_w;
    a.distill_min_clamp = a.distill_token_clip = a.distill_is_clip = NAN;
    a.topk_ids = d_ids;
    a.topk_teacher_log_prob = d_tlp;
    a.topk_k = K;
    a.topk_kl_mode = RELAX_AMD_OPD_JSD;
    a.topk_norm_mode = RELAX_AMD_OPD_NORM_TRUNC;
    a.topk_jsd_alpha = 0.0f;
    a.topk_kl = d_tkl;
    a.topk_grad = d_tgrad;
    CHECK_LIB(relax_amd_actor_step_fused(d_logits, RELAX_AMD_F32, N, V, V, NULL, (const int32_t*)d_sid,
                                         (const int64_t*)d_tokens, 1.0f, &a, 1.0f, d_lp3, d_ent3, d_lse, d_spx, d_grad, V,
                                         stream));
    CHECK_LIB(relax_amd_sparse_row_add(d_grad, RELAX_AMD_F32, N, V, V, NULL, (const int64_t*)d_ids, d_tgrad, K, NULL, NULL,
                                       1.0f, stream));
    a.log_prob = d_lp3; /* the loss value and metrics of the policy terms, from the step's log-probs */
    a.entropy = d_ent3;
    CHECK_LIB(relax_amd_policy_loss(&a, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    float lp3[N], tkl[N], met[RELAX_AMD_NUM_METRICS];
    CHECK_HIP(hipMemcpy(lp3, d_lp3, sizeof lp3, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(tkl, d_tkl, sizeof tkl, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(met, d_met, sizeof met, hipMemcpyDeviceToHost));
    CHECK_HIP(hipMemcpy(grad, d_grad, sizeof grad, hipMemcpyDeviceToHost));
    ok &= close_enough("fused pg loss", 0, met[RELAX_AMD_M_PG_LOSS], -(1.0 - 2.0 + 0.5) / 3.0, 2e-6);
    for (int i = 0; i < N; ++i) {
      double z = 0;
      for (int v = 0; v < V; ++v) z += exp((double)logits[i][v]);
      const double lse = log(z);
      ok &= close_enough("fused log_prob", i, lp3[i], lp[i], 0.0);
      double want_kl = 0, dk[K];
      for (int k = 0; k < K; ++k) {
        const double s = logits[i][ids[i][k]] - lse;
        want_kl += exp(s) * (s - teacher_lp[i][k]);
        dk[k] = exp(s) * (s - teacher_lp[i][k] + 1.0);
      }
      ok &= close_enough("fused top-K KL", i, tkl[i], want_kl, 2e-6);
      for (int v = 0; v < V; ++v) {
        const double p = exp(logits[i][v] - lse);
        double want = -(adv[i] / 3.0) * ((v == tokens[i]) - p);
        for (int k = 0; k < K; ++k) want += w * dk[k] * ((v == ids[i][k]) - p);
        ok &= close_enough("fused dlogits", i * V + v, grad[i][v], want, 2e-6);
      }
    }
  }
  /* error path: the library reports instead of launching */
  if (relax_amd_logprob_entropy_fwd(d_logits, 99, N, V, V, NULL, (const int64_t*)d_tokens, 1.0f, d_lp, d_ent, d_lse,
                                    d_spx, stream) == RELAX_AMD_OK) {
    fprintf(stderr, "an unknown dtype code was accepted\n");
    ok = 0;
  }
  printf(ok ? "abi_client ok\n" : "abi_client FAILED\n");
  return ok ? 0 : 1;
}
