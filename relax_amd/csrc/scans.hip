// Per-sequence reverse recurrences over the packed response layout, and the REINFORCE++ population normaliser.
//
//   reinforce_pp_returns  <- get_reinforce_plus_plus_returns   (relax/utils/training/ppo_utils.py:708-804, cp_size 1)
//   gae                   <- get_advantages_and_returns / vanilla_gae   (ppo_utils.py:846-906, 1026-1047)
//   masked_normalize      <- distributed_masked_normalize   (relax/utils/distributed_utils.py:161-213, one rank)
//
// Both recurrences are y_t = x_t + a * y_{t+1}.  One wave owns one sequence and walks it from the end in 64-token
// chunks: the chunk is loaded coalesced, lane 0 runs the 64 dependent steps in the reference's order (a multiply and
// an add, each rounded on its own, so the result is bit-identical to the sequential Python loop), and the chunk is
// stored coalesced.  The data is a few hundred KB; what matters is one launch instead of one Python iteration per
// token.
#include "device_utils.h"
#include "relax_amd.h"

// The recurrences must round the multiply and the add separately, as the reference's tensor arithmetic does: no
// fused multiply-add contraction anywhere in this file.
#pragma clang fp contract(off)

namespace relax_amd {

// Written out here, below the pragma (operations inside library inline functions keep the contraction setting of the
// header they come from and would fuse again after inlining).
template <typename F>
__device__ __forceinline__ F mul_rn(F a, F b) {
  return a * b;
}
template <typename F>
__device__ __forceinline__ F add_rn(F a, F b) {
  return a + b;
}

// G_t = r_t + gamma * G_{t+1} with r_t = -kl_coef * kl_t on valid tokens (0 elsewhere; a masked NaN never enters) and
// the sequence reward added at the last valid token; returns are zero outside the mask and for fully masked sequences.
template <typename F>
__global__ __launch_bounds__(kWave) void reinforce_pp_returns_kernel(const F* __restrict__ kl,
                                                                     const F* __restrict__ mask,
                                                                     const F* __restrict__ rewards,
                                                                     const int64_t* __restrict__ cu, F kl_coef,
                                                                     F gamma, F* __restrict__ out) {
  __shared__ F xs[kWave], ys[kWave];
  const int lane = threadIdx.x;
  const int64_t seq = blockIdx.x, beg = cu[seq], len = cu[seq + 1] - cu[seq];
  long long last = -1;
  for (int64_t j = lane; j < len; j += kWave)
    if (mask[beg + j] != F(0)) last = j;
  wave_butterfly([&](auto o) {
    const long long other = lane_xor<decltype(o)::value>(last);
    last = other > last ? other : last;
  });
  if (last < 0) {
    for (int64_t j = lane; j < len; j += kWave) out[beg + j] = F(0);
    return;
  }
  const F reward = rewards[seq];
  F run = F(0);
  for (int64_t end = len; end > 0; end -= kWave) {
    const int64_t base = end > kWave ? end - kWave : 0;
    const int cnt = int(end - base);
    bool valid = false;
    if (lane < cnt) {
      valid = mask[beg + base + lane] != F(0);
      F x = mul_rn<F>(-kl_coef, valid ? kl[beg + base + lane] : F(0));
      if (base + lane == last) x = add_rn<F>(x, reward);
      xs[lane] = x;
    }
    __syncthreads();
    if (lane == 0) {
      for (int j = cnt - 1; j >= 0; --j) {
        run = add_rn<F>(xs[j], mul_rn<F>(gamma, run));
        ys[j] = run;
      }
    }
    __syncthreads();
    if (lane < cnt) out[beg + base + lane] = valid ? ys[lane] : F(0);
  }
}

// delta_t = r_t + gamma * V_{t+1} - V_t (V past the end = 0), A_t = delta_t + (gamma*lambda) * A_{t+1}, R_t = A_t + V_t
template <typename F>
__global__ __launch_bounds__(kWave) void gae_kernel(const F* __restrict__ values, const F* __restrict__ rewards,
                                                    const int64_t* __restrict__ cu, F gamma, F gamma_lambda,
                                                    F* __restrict__ adv, F* __restrict__ ret) {
  __shared__ F xs[kWave], ys[kWave];
  const int lane = threadIdx.x;
  const int64_t seq = blockIdx.x, beg = cu[seq], len = cu[seq + 1] - cu[seq];
  F run = F(0);
  for (int64_t end = len; end > 0; end -= kWave) {
    const int64_t base = end > kWave ? end - kWave : 0;
    const int cnt = int(end - base);
    F v = F(0);
    if (lane < cnt) {
      const int64_t t = base + lane;
      v = values[beg + t];
      const F next = t + 1 < len ? values[beg + t + 1] : F(0);
      xs[lane] = add_rn<F>(add_rn<F>(rewards[beg + t], mul_rn<F>(gamma, next)), -v);
    }
    __syncthreads();
    if (lane == 0) {
      for (int j = cnt - 1; j >= 0; --j) {
        run = add_rn<F>(xs[j], mul_rn<F>(gamma_lambda, run));
        ys[j] = run;
      }
    }
    __syncthreads();
    if (lane < cnt) {
      adv[beg + base + lane] = ys[lane];
      ret[beg + base + lane] = add_rn<F>(ys[lane], v);
    }
  }
}

// Population moments over mask != 0 (ddof = 0), output zero outside the mask.  One workgroup: the vectors are at most
// a few hundred thousand elements and the three passes need the previous pass's total anyway.
constexpr int kNormThreads = 1024;
template <typename F>
__global__ __launch_bounds__(kNormThreads) void masked_normalize_kernel(const F* __restrict__ x,
                                                                        const F* __restrict__ mask, int64_t n,
                                                                        F variance_floor, F* __restrict__ out,
                                                                        F* __restrict__ stats) {
  __shared__ double part[kNormThreads / kWave];
  double s = 0.0, c = 0.0;
  for (int64_t i = threadIdx.x; i < n; i += kNormThreads)
    if (mask[i] != F(0)) {
      s += double(x[i]);
      c += 1.0;
    }
  s = block_sum<kNormThreads>(s, part);
  c = block_sum<kNormThreads>(c, part);
  const F count = F(c), safe = count < F(1) ? F(1) : count;
  const F mean = F(s) / safe;
  double q = 0.0;
  for (int64_t i = threadIdx.x; i < n; i += kNormThreads)
    if (mask[i] != F(0)) {
      const F d = x[i] - mean;
      q += double(d * d);
    }
  q = block_sum<kNormThreads>(q, part);
  F var = F(q) / safe;
  if (var < F(0)) var = F(0);
  const F floored = var < variance_floor ? variance_floor : var;
  const F rstd = F(1) / F(sqrt(double(floored)));
  for (int64_t i = threadIdx.x; i < n; i += kNormThreads) out[i] = mask[i] != F(0) ? (x[i] - mean) * rstd : F(0);
  if (threadIdx.x == 0) {
    stats[0] = mean;
    stats[1] = var;
    stats[2] = count;
  }
}

}  // namespace relax_amd

using namespace relax_amd;

static int scan_check(const char* what, int dtype, int64_t n_samples) {
  if (dtype != RELAX_AMD_F32 && dtype != RELAX_AMD_F64) {
    set_error("%s: dtype must be F32 or F64 (got %d)", what, dtype);
    return RELAX_AMD_EINVAL;
  }
  if (n_samples < 0 || n_samples > 2147483647LL) {
    set_error("%s: bad n_samples=%lld", what, (long long)n_samples);
    return RELAX_AMD_EINVAL;
  }
  return RELAX_AMD_OK;
}

extern "C" int relax_amd_reinforce_pp_returns(const void* kl, const void* mask, const void* rewards, int dtype,
                                              const int64_t* cu_resp, int64_t n_samples, double kl_coef, double gamma,
                                              void* returns, void* stream) {
  if (int rc = scan_check("reinforce_pp_returns", dtype, n_samples)) return rc;
  if (n_samples == 0) return RELAX_AMD_OK;
  if (!kl || !mask || !rewards || !cu_resp || !returns) {
    set_error("reinforce_pp_returns: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(n_samples));
  if (dtype == RELAX_AMD_F32)
    hipLaunchKernelGGL(reinforce_pp_returns_kernel<float>, grid, dim3(kWave), 0, s, static_cast<const float*>(kl),
                       static_cast<const float*>(mask), static_cast<const float*>(rewards), cu_resp, float(kl_coef),
                       float(gamma), static_cast<float*>(returns));
  else
    hipLaunchKernelGGL(reinforce_pp_returns_kernel<double>, grid, dim3(kWave), 0, s, static_cast<const double*>(kl),
                       static_cast<const double*>(mask), static_cast<const double*>(rewards), cu_resp, kl_coef, gamma,
                       static_cast<double*>(returns));
  return check_launch("reinforce_pp_returns");
}

extern "C" int relax_amd_gae(const void* values, const void* rewards, int dtype, const int64_t* cu_resp,
                             int64_t n_samples, double gamma, double lambd, void* advantages, void* returns,
                             void* stream) {
  if (int rc = scan_check("gae", dtype, n_samples)) return rc;
  if (n_samples == 0) return RELAX_AMD_OK;
  if (!values || !rewards || !cu_resp || !advantages || !returns) {
    set_error("gae: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(n_samples));
  if (dtype == RELAX_AMD_F32)
    hipLaunchKernelGGL(gae_kernel<float>, grid, dim3(kWave), 0, s, static_cast<const float*>(values),
                       static_cast<const float*>(rewards), cu_resp, float(gamma), float(gamma * lambd),
                       static_cast<float*>(advantages), static_cast<float*>(returns));
  else
    hipLaunchKernelGGL(gae_kernel<double>, grid, dim3(kWave), 0, s, static_cast<const double*>(values),
                       static_cast<const double*>(rewards), cu_resp, gamma, gamma * lambd,
                       static_cast<double*>(advantages), static_cast<double*>(returns));
  return check_launch("gae");
}

extern "C" int relax_amd_masked_normalize(const void* values, const void* mask, int dtype, int64_t n,
                                          double variance_floor, void* out, void* stats, void* stream) {
  if (int rc = scan_check("masked_normalize", dtype, 0)) return rc;
  if (n < 0 || !(variance_floor > 0.0)) {
    set_error("masked_normalize: n must be >= 0 and variance_floor positive");
    return RELAX_AMD_EINVAL;
  }
  if (!stats || (n > 0 && (!values || !mask || !out))) {
    set_error("masked_normalize: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == RELAX_AMD_F32)
    hipLaunchKernelGGL(masked_normalize_kernel<float>, dim3(1), dim3(kNormThreads), 0, s,
                       static_cast<const float*>(values), static_cast<const float*>(mask), n, float(variance_floor),
                       static_cast<float*>(out), static_cast<float*>(stats));
  else
    hipLaunchKernelGGL(masked_normalize_kernel<double>, dim3(1), dim3(kNormThreads), 0, s,
                       static_cast<const double*>(values), static_cast<const double*>(mask), n, variance_floor,
                       static_cast<double*>(out), static_cast<double*>(stats));
  return check_launch("masked_normalize");
}
