// Group-normalised rewards (GRPO mean/std, RLOO leave-one-out), per-sample -> per-token broadcast, and masked
// whitening.  These touch kilobytes, so they are launch-latency bound; the design goal is exact reference arithmetic
// (fp32 like torch, unbiased std, +1e-6) and fixed summation order, not bandwidth.
#include "device_utils.h"
#include "relax_amd.h"

namespace relax_amd {

// One thread per sample; each thread scans all samples in position order and combines the members of its own
// group.  O(n^2) on n <= a few thousand rewards; every member of a group computes bit-identical statistics.
// Arithmetic of relax/utils/utils.py:219-236 and relax/utils/training/ppo_utils.py:703-705.
template <typename F>
__global__ __launch_bounds__(256) void group_rewards_kernel(const F* __restrict__ r, const int32_t* __restrict__ g,
                                                            int64_t n, int mode, F* __restrict__ out,
                                                            int32_t* __restrict__ count) {
  const int64_t i = blockIdx.x * 256LL + threadIdx.x;
  if (i >= n) return;
  const int32_t gi = g[i];
  F sum = 0;
  int32_t cnt = 0;
  for (int64_t j = 0; j < n; ++j)
    if (g[j] == gi) {
      sum += r[j];
      ++cnt;
    }
  const F mean = sum / F(cnt);
  F v = r[i] - mean;
  if (mode == RELAX_AMD_GROUP_CENTER_STD) {
    // torch.std of the centred group: unbiased, computed around the centred group's own mean
    F csum = 0;
    for (int64_t j = 0; j < n; ++j)
      if (g[j] == gi) csum += r[j] - mean;
    const F cmean = csum / F(cnt);
    F ss = 0;
    for (int64_t j = 0; j < n; ++j)
      if (g[j] == gi) {
        const F d = (r[j] - mean) - cmean;
        ss += d * d;
      }
    const F sd = sqrt(ss / F(cnt - 1));  // cnt == 1 gives NaN, as torch.std does
    v = v / (sd + F(1e-6));
  } else if (mode == RELAX_AMD_GROUP_RLOO) {
    v = (F(cnt) / F(cnt - 1)) * v;
  }
  out[i] = v;
  if (count) count[i] = cnt;
}

__global__ __launch_bounds__(256) void broadcast_per_sample_kernel(const float* __restrict__ per_sample,
                                                                   const int64_t* __restrict__ cu,
                                                                   float* __restrict__ out) {
  const int64_t i = blockIdx.x;
  const float v = per_sample[i];
  for (int64_t t = cu[i] + threadIdx.x; t < cu[i + 1]; t += 256) out[t] = v;
}

constexpr int kWhitenThreads = 256;
constexpr int64_t kWhitenPerBlock = 256 * 16;

__global__ __launch_bounds__(kWhitenThreads) void whiten_partial_kernel(const float* __restrict__ x,
                                                                        const float* __restrict__ m, int64_t n,
                                                                        double* __restrict__ partials) {
  __shared__ double red[kWhitenThreads / kWave];
  const int64_t base = blockIdx.x * kWhitenPerBlock;
  double s1 = 0, s2 = 0, s0 = 0;
  for (int64_t k = threadIdx.x; k < kWhitenPerBlock; k += kWhitenThreads) {
    const int64_t t = base + k;
    if (t < n) {
      const float xv = x[t], mv = m[t];
      s1 += double(xv * mv);
      s2 += double((xv * xv) * mv);
      s0 += double(mv);
    }
  }
  s1 = block_sum<kWhitenThreads>(s1, red);
  s2 = block_sum<kWhitenThreads>(s2, red);
  s0 = block_sum<kWhitenThreads>(s0, red);
  if (threadIdx.x == 0) {
    partials[3 * blockIdx.x + 0] = s1;
    partials[3 * blockIdx.x + 1] = s2;
    partials[3 * blockIdx.x + 2] = s0;
  }
}

// relax/utils/distributed_utils.py:128-153: the three sums are rounded to fp32 before the statistics.
__global__ __launch_bounds__(kWave) void whiten_stats_kernel(const double* __restrict__ partials, int64_t blocks,
                                                             float epsilon, float* __restrict__ stats) {
  if (threadIdx.x != 0) return;
  double s1 = 0, s2 = 0, s0 = 0;
  for (int64_t b = 0; b < blocks; ++b) {
    s1 += partials[3 * b];
    s2 += partials[3 * b + 1];
    s0 += partials[3 * b + 2];
  }
  const float f1 = float(s1), f2 = float(s2), f0 = float(s0);
  const float mean = f1 / f0;
  float var = f2 / f0 - mean * mean;
  if (f0 >= 2.0f) var = var * (f0 / (f0 - 1.0f));
  stats[0] = f1;
  stats[1] = f2;
  stats[2] = f0;
  stats[3] = 1.0f / sqrtf(var + epsilon);
}

__global__ __launch_bounds__(256) void whiten_apply_kernel(const float* __restrict__ x, int64_t n,
                                                           const float* __restrict__ stats, int shift_mean,
                                                           float* __restrict__ out) {
  const float mean = stats[0] / stats[2], rstd = stats[3];
  for (int64_t t = blockIdx.x * 256LL + threadIdx.x; t < n; t += int64_t(gridDim.x) * 256) {
    float v = (x[t] - mean) * rstd;
    if (!shift_mean) v += mean;
    out[t] = v;
  }
}

}  // namespace relax_amd

using namespace relax_amd;

extern "C" int relax_amd_group_rewards(const void* rewards, int dtype, const int32_t* group_index, int64_t n,
                                       int32_t mode, void* out, int32_t* group_count, void* stream) {
  if (n < 0 || n > (1LL << 20)) {
    set_error("group_rewards: n=%lld outside [0, 2^20]", (long long)n);
    return RELAX_AMD_EINVAL;
  }
  if (mode < RELAX_AMD_GROUP_CENTER || mode > RELAX_AMD_GROUP_RLOO) {
    set_error("group_rewards: unknown mode %d", mode);
    return RELAX_AMD_EINVAL;
  }
  if (dtype != RELAX_AMD_F32 && dtype != RELAX_AMD_F64) {
    set_error("group_rewards: dtype must be F32 or F64 (got %d)", dtype);
    return RELAX_AMD_EINVAL;
  }
  if (n == 0) return RELAX_AMD_OK;
  if (!rewards || !group_index || !out) {
    set_error("group_rewards: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  const dim3 grid(static_cast<unsigned>((n + 255) / 256));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == RELAX_AMD_F32)
    hipLaunchKernelGGL(group_rewards_kernel<float>, grid, dim3(256), 0, s, static_cast<const float*>(rewards),
                       group_index, n, mode, static_cast<float*>(out), group_count);
  else
    hipLaunchKernelGGL(group_rewards_kernel<double>, grid, dim3(256), 0, s, static_cast<const double*>(rewards),
                       group_index, n, mode, static_cast<double*>(out), group_count);
  return check_launch("group_rewards");
}

extern "C" int relax_amd_broadcast_per_sample(const float* per_sample, const int64_t* cu_resp, int64_t n_samples,
                                              float* out, void* stream) {
  if (n_samples < 0 || n_samples > 2147483647LL) {
    set_error("broadcast_per_sample: bad n_samples");
    return RELAX_AMD_EINVAL;
  }
  if (n_samples == 0) return RELAX_AMD_OK;
  if (!per_sample || !cu_resp || !out) {
    set_error("broadcast_per_sample: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipLaunchKernelGGL(broadcast_per_sample_kernel, dim3(static_cast<unsigned>(n_samples)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), per_sample, cu_resp, out);
  return check_launch("broadcast_per_sample");
}

extern "C" int64_t relax_amd_whiten_partials(int64_t n) {
  return n <= 0 ? 0 : (n + kWhitenPerBlock - 1) / kWhitenPerBlock;
}

extern "C" int relax_amd_masked_whiten(const float* values, const float* mask, int64_t n, int32_t shift_mean,
                                       float epsilon, double* partials, float* stats, float* out, void* stream) {
  if (n <= 0) {
    set_error("masked_whiten: n must be > 0");
    return RELAX_AMD_EINVAL;
  }
  if (!values || !mask || !partials || !stats || !out) {
    set_error("masked_whiten: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t blocks = relax_amd_whiten_partials(n);
  hipLaunchKernelGGL(whiten_partial_kernel, dim3(static_cast<unsigned>(blocks)), dim3(kWhitenThreads), 0, s, values,
                     mask, n, partials);
  int rc = check_launch("whiten_partial");
  if (rc) return rc;
  hipLaunchKernelGGL(whiten_stats_kernel, dim3(1), dim3(kWave), 0, s, partials, blocks, epsilon, stats);
  rc = check_launch("whiten_stats");
  if (rc) return rc;
  const unsigned grid = static_cast<unsigned>((n + 255) / 256 > 8192 ? 8192 : (n + 255) / 256);
  hipLaunchKernelGGL(whiten_apply_kernel, dim3(grid), dim3(256), 0, s, values, n, stats, int(shift_mean), out);
  return check_launch("whiten_apply");
}
