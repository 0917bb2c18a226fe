// Online-softmax state and update rules shared by the reverse-KL kernels (reverse_kl.hip, reverse_kl_resident.hip, reverse_kl_split.hip).
#pragma once

#include "device_utils.h"

namespace relax_amd {

constexpr int kKlThreads = 256;
constexpr int kKlUnroll = 2;

struct KlState {
  float ms, ss, us, mt, st;
};

template <int K>
__device__ __forceinline__ void absorb_pair(const float (&xs)[K], const float (&xt)[K], KlState& q) {
  float smax = xs[0], tmax = xt[0];
#pragma unroll
  for (int i = 1; i < K; ++i) {
    smax = fmaxf(smax, xs[i]);
    tmax = fmaxf(tmax, xt[i]);
  }
  const float sm = smax * kLog2e, tm = tmax * kLog2e;
  if (sm > q.ms) {
    const float sc = fast_exp2(q.ms - sm);
    q.ss *= sc;
    q.us *= sc;
    q.ms = sm;
  }
  if (tm > q.mt) {
    q.st *= fast_exp2(q.mt - tm);
    q.mt = tm;
  }
#pragma unroll
  for (int i = 0; i < K; ++i) {
    const float es = fast_exp2(fmaf(xs[i], kLog2e, -q.ms));
    const float et = fast_exp2(fmaf(xt[i], kLog2e, -q.mt));
    q.ss += es;
    q.us = fmaf(es, xs[i] - xt[i], q.us);
    q.st += et;
  }
}

__device__ __forceinline__ void merge_kl(KlState& a, const KlState& b) {
  const float ms = fmaxf(a.ms, b.ms), mt = fmaxf(a.mt, b.mt);
  const float fa = fast_exp2(a.ms - ms), fb = fast_exp2(b.ms - ms);
  // the fused multiply-adds spelled out: left as a * fa + b * fb the compiler picks which product to fuse by
  // context, and the kernels that share this rule would differ in the last bit
  a.ss = fmaf(a.ss, fa, b.ss * fb);
  a.us = fmaf(a.us, fa, b.us * fb);
  a.st = fmaf(a.st, fast_exp2(a.mt - mt), b.st * fast_exp2(b.mt - mt));
  a.ms = ms;
  a.mt = mt;
}

// the row's results from its merged state: KL(student || teacher) = sum p_s (x_s - x_t) - lse_s + lse_t
struct KlRow {
  float kl, lse_s, lse_t;
};
__device__ __forceinline__ KlRow kl_finish(const KlState& q) {
  KlRow r;
  r.lse_s = fmaf(q.ms, kLn2, logf(q.ss));
  r.lse_t = fmaf(q.mt, kLn2, logf(q.st));
  r.kl = q.us / q.ss - r.lse_s + r.lse_t;
  return r;
}

}  // namespace relax_amd
