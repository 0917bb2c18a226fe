// Fused actor step: log-prob + entropy forward, per-token policy-loss coefficients and dlogits backward in ONE launch,
// one workgroup per logits row.
//
// The workgroup scans its row once with ordinary (cached) loads to get the online-softmax statistics, thread 0
// evaluates the token's loss terms (the same token_terms() the stand-alone policy-loss kernel uses) and broadcasts the
// row's gradient constants, and the workgroup immediately walks the row a second time to emit dlogits with
// non-temporal stores.  The second walk starts microseconds after the first, while only a few hundred rows are in
// flight on the whole device, so it is served by the L2 / memory-side cache instead of HBM: HBM sees one read and one
// write per row (2*V*s bytes per token) instead of the 3*V*s of separate forward and backward launches, and unlike a
// register-resident row this works for any row length with many workgroups per CU overlapping each other's phases.
//
// Rows that score no token, and tokens whose loss masks are both zero (every loss term, metric and gradient of such
// a token is multiplied by the mask), are never read: their dlogits row is zero-filled and their per-token outputs
// are written as zeros.
//
// This fusion is possible whenever d loss / d log_prob of a token depends only on that token (PPO-clip, CISPO, RLOO,
// SAPO, KL penalties, entropy bonus, TIS weights) and the per-sample denominators are known up front (they only
// depend on the masks).  GSPO and OPSM couple the tokens of a sequence and use the two-launch path.
//
// Replaces, for one micro-batch, _VocabParallelLogProbEntropy.forward + .backward
// (relax/utils/training/ppo_utils.py:481-629) and the per-token part of policy_loss_function
// (relax/backends/megatron/loss.py:961-1100).
#include "device_utils.h"
#include "loss_math.h"
#include "opd_topk_math.h"
#include "relax_amd.h"
#include "row_scan.h"

#include <cstdlib>
#include <cstring>

#include "actor_step_resident.h"

namespace relax_amd {

template <typename T, bool VEC, int THREADS>
__device__ __forceinline__ void fused_zero_row(T* __restrict__ d, int64_t vocab) {
  if (VEC) {
    constexpr int VN = Row<T>::kPerVec;
    u32x4* dv = reinterpret_cast<u32x4*>(d);
    const int64_t nvec = vocab / VN;
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int64_t i = threadIdx.x; i < nvec; i += THREADS) store_stream(dv + i, z);
    for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += THREADS) Row<T>::store1(d + e, 0.f);
  } else {
    for (int64_t e = threadIdx.x; e < vocab; e += THREADS) Row<T>::store1(d + e, 0.f);
  }
}

template <typename T, bool VEC, int THREADS>
__global__ __launch_bounds__(THREADS) void actor_step_fused_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t vocab, const int32_t* __restrict__ token_of_row,
    const int32_t* __restrict__ sample_ids, const int64_t* __restrict__ targets, float c, float inv_t,
    relax_amd_policy_loss_args a, float grad_scale, float* __restrict__ log_prob, float* __restrict__ entropy,
    float* __restrict__ lse_out, float* __restrict__ spx_out, T* __restrict__ dlogits, int64_t d_stride) {
  __shared__ float wave_state[THREADS / kWave][3];
  __shared__ float bc[5];
  __shared__ int64_t bc_target;
  __shared__ float topk_stage[kTopkStageFloats];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  T* d = dlogits + row * d_stride;
  const int64_t tok = token_of_row ? int64_t(token_of_row[row]) : row;
  bool live = tok >= 0;
  if (live) {
    const float m = a.loss_mask[tok];
    const float mp = a.pg_loss_mask ? a.pg_loss_mask[tok] : m;
    live = !(m == 0.f && mp == 0.f) || a.read_masked_rows != 0;
  }
  if (!live) {
    fused_zero_row<T, VEC, THREADS>(d, vocab);
    if (tok >= 0 && tid == 0) {
      log_prob[tok] = 0.f;
      entropy[tok] = 0.f;
      lse_out[tok] = 0.f;
      spx_out[tok] = 0.f;
      a.coef_log_prob[tok] = 0.f;
      if (a.coef_entropy) a.coef_entropy[tok] = 0.f;
    }
    return;
  }
  const T* x = logits + row * row_stride;
  // thread 0 fetches the token's scalars now; they arrive while the row is scanned
  TokenInputs in{};
  float x_target = 0.f, den = 1.f, pg_den = 1.f;
  int64_t tg = -1;
  if (tid == 0) {
    in = load_token_inputs(a, tok);
    tg = targets[tok];
    if (tg >= 0 && tg < vocab) x_target = Row<T>::load1(x + tg);
    const int32_t sid = sample_ids ? sample_ids[tok] : 0;
    den = a.sample_denom ? a.sample_denom[sid] : 1.0f;
    pg_den = a.pg_sample_denom ? a.pg_sample_denom[sid] : den;
  }
  // the first wave's gathers for the top-K distillation signal, when configured, likewise
  TopkGather gathered{};
  TopkRowShape topk_shape{};
  if (a.topk_ids && tid < kWave) {
    gathered = topk_gather<T>(a, x, vocab, tok, tid);
    topk_shape = topk_row_shape(a, tok);
  }
  // pass 1: cached loads, the row stays in L2 / the memory-side cache for pass 2
  SoftmaxAcc st = scan_row<T, VEC, false, THREADS>(x, vocab, c);
  scan_block_merge<THREADS>(st, wave_state);
  if (tid < kWave) {  // the first wave; thread 0 holds the merged state and the token's scalars
    float lse = 0.f, spx = 0.f, ent = 0.f, lp = 0.f;
    if (tid == 0) {
      scan_finish(st, x_target, tg >= 0 && tg < vocab, inv_t, lse, spx, ent, lp);
      log_prob[tok] = lp;
      entropy[tok] = ent;
      lse_out[tok] = lse;
      spx_out[tok] = spx;
    }
    // the top-K distillation signal, when configured: K gathered logits of this row against the log-sum-exp just found
    float g_topk = 0.f;
    if (a.topk_ids) {
      const float lp0 = lane_value(lp);
      g_topk = topk_distill_row(a, gathered, topk_shape, tok, lane_value(lse), inv_t, lp0,
                                lane_value(in.has_old ? in.old_lp : lp), lane_value(in.extra_lp), tid,
                                topk_stage);
    }
    if (tid == 0) {
      const TokenResult tr = token_terms(a, in, lp, ent, false, 0.f, den, pg_den);
      a.coef_log_prob[tok] = tr.coef_lp;
      if (a.coef_entropy) a.coef_entropy[tok] = tr.coef_ent;
      const float glp = tr.coef_lp * grad_scale, gh = tr.coef_ent * grad_scale;
      const float gsm = glp + g_topk * grad_scale;  // what the row's softmax is subtracted with
      const float b = gh * inv_t;
      bc[0] = -lse * kLog2e;           // k0: p = exp2(x*c + k0)
      bc[1] = -gsm * inv_t + b * spx;  // a0
      bc[2] = -b * inv_t;              // a1: d = p * (a0 + a1*x)
      bc[3] = glp * inv_t;             // added at the target
      bc[4] = (gsm == 0.f && glp == 0.f && gh == 0.f) ? 1.f : 0.f;
      bc_target = tg;
    }
  }
  __syncthreads();
  const float k0 = bc[0], a0 = bc[1], a1 = bc[2], hot = bc[3];
  tg = bc_target;
  if (bc[4] != 0.f) {
    fused_zero_row<T, VEC, THREADS>(d, vocab);
    return;
  }
  // pass 2: last use of the row (non-temporal loads), dlogits streamed out
  if (VEC) {
    constexpr int VN = Row<T>::kPerVec;
    const u32x4* xv = reinterpret_cast<const u32x4*>(x);
    u32x4* dv = reinterpret_cast<u32x4*>(d);
    const int64_t nvec = vocab / VN;
    const int64_t tvec = (tg >= 0 && tg < nvec * VN) ? tg / VN : -1;
    const int tsub = int(tg % VN);
    // The row is walked from its end to its beginning: what the scan read last is what the caches still hold, so the
    // second walk starts where the first one stopped.  The lane's share is the scan's: `nfull` batches of kScanUnroll
    // vectors at a stride of THREADS, then `nsingle` single vectors, then tail elements.
    const int64_t nfull = nvec > int64_t(kScanUnroll - 1) * THREADS + tid
                              ? (nvec - int64_t(kScanUnroll - 1) * THREADS - tid - 1) / (int64_t(kScanUnroll) * THREADS) + 1
                              : 0;
    const int64_t single0 = int64_t(tid) + nfull * kScanUnroll * THREADS;
    const int64_t nsingle = single0 < nvec ? (nvec - single0 - 1) / THREADS + 1 : 0;
    for (int64_t e = nvec * VN + tid; e < vocab; e += THREADS) {
      const float xe = Row<T>::load1(x + e);
      float g = fast_exp2(fmaf(xe, c, k0)) * fmaf(xe, a1, a0);
      if (e == tg) g += hot;
      Row<T>::store1(d + e, g);
    }
    for (int64_t q = nsingle - 1; q >= 0; --q) {
      const int64_t i = single0 + q * THREADS;
      float v[VN];
      Row<T>::unpack(load_stream(xv + i), v);
#pragma unroll
      for (int k = 0; k < VN; ++k) v[k] = fast_exp2(fmaf(v[k], c, k0)) * fmaf(v[k], a1, a0);
      if (i == tvec) {
#pragma unroll
        for (int k = 0; k < VN; ++k)
          if (k == tsub) v[k] += hot;
      }
      store_stream(dv + i, Row<T>::pack(v));
    }
    for (int64_t b = nfull - 1; b >= 0; --b) {
      const int64_t i = int64_t(tid) + b * kScanUnroll * THREADS;
      u32x4 raw[kScanUnroll];
#pragma unroll
      for (int u = kScanUnroll - 1; u >= 0; --u) raw[u] = load_stream(xv + i + int64_t(u) * THREADS);
#pragma unroll
      for (int u = kScanUnroll - 1; u >= 0; --u) {
        float v[VN];
        Row<T>::unpack(raw[u], v);
#pragma unroll
        for (int k = 0; k < VN; ++k) v[k] = fast_exp2(fmaf(v[k], c, k0)) * fmaf(v[k], a1, a0);
        if (i + int64_t(u) * THREADS == tvec) {
#pragma unroll
          for (int k = 0; k < VN; ++k)
            if (k == tsub) v[k] += hot;
        }
        store_stream(dv + i + int64_t(u) * THREADS, Row<T>::pack(v));
      }
    }
  } else {
    for (int64_t e = tid; e < vocab; e += THREADS) {
      const float xe = Row<T>::load1(x + e);
      float g = fast_exp2(fmaf(xe, c, k0)) * fmaf(xe, a1, a0);
      if (e == tg) g += hot;
      Row<T>::store1(d + e, g);
    }
  }
}

static int device_compute_units() {
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return 256;
  return cus;
}

template <typename T>
static int dispatch_fused(const void* logits, int64_t n_rows, int64_t vocab, int64_t stride,
                          const int32_t* token_of_row, const int32_t* sample_ids, const int64_t* targets, float inv_t,
                          const relax_amd_policy_loss_args& a, float grad_scale, float* lp, float* ent, float* lse,
                          float* spx, void* dlogits, int64_t d_stride, hipStream_t s) {
  const bool vec = aligned16(logits) && aligned16(dlogits) && (stride * int64_t(sizeof(T))) % 16 == 0 &&
                   (d_stride * int64_t(sizeof(T))) % 16 == 0;
  const T* x = static_cast<const T*>(logits);
  T* d = static_cast<T*>(dlogits);
  dim3 grid(static_cast<unsigned>(n_rows));
  // relax_amd_set_kernel_choice: TWO_WALK keeps every row on the two-walk kernel (second walk out of cache); RESIDENT
  // fails for rows the register-resident kernel is not built for
  const int choice = kernel_choice();
  if (vec && choice == RELAX_AMD_KERNEL_AUTO) {  // one-shot workgroups sharing each row, where built
    const int rc = launch_actor_step_split<T>(x, stride, vocab, n_rows, token_of_row, sample_ids, targets, inv_t, a,
                                              grad_scale, lp, ent, lse, spx, d, d_stride, s);
    if (rc != RELAX_AMD_EUNSUPPORTED) return rc;
  }
  if (vec && choice != RELAX_AMD_KERNEL_TWO_WALK) {
    const int rc = launch_actor_step_resident<T>(x, stride, vocab, n_rows, token_of_row, sample_ids, targets, inv_t, a,
                                                 grad_scale, lp, ent, lse, spx, d, d_stride, device_compute_units(), s);
    if (rc != RELAX_AMD_EUNSUPPORTED) return rc;  // launched (or failed to): otherwise the row length is not built
    if constexpr (sizeof(T) == 4) {  // long fp32 rows: resident as their upper halves where those are exact
      const int rcw = launch_actor_step_resident_wide(x, stride, vocab, n_rows, token_of_row, sample_ids, targets,
                                                      inv_t, a, grad_scale, lp, ent, lse, spx, d, d_stride,
                                                      device_compute_units(), s);
      if (rcw != RELAX_AMD_EUNSUPPORTED) return rcw;
    }
  }
  if (choice == RELAX_AMD_KERNEL_RESIDENT) {
    set_error("actor_step_fused: kernel choice RESIDENT, but no register-resident kernel is built for "
              "rows of %lld elements of this type and alignment", (long long)vocab);
    return RELAX_AMD_EUNSUPPORTED;
  }
#define RELAX_AMD_FUSED(V, TH)                                                                                     \
  hipLaunchKernelGGL((actor_step_fused_kernel<T, V, TH>), grid, dim3(TH), 0, s, x, stride, vocab, token_of_row,       \
                     sample_ids, targets, inv_t * kLog2e, inv_t, a, grad_scale, lp, ent, lse, spx, d, d_stride)
  if (!vec) {
    RELAX_AMD_FUSED(false, 256);
  } else {
    switch (scan_threads(vocab, Row<T>::kPerVec)) {
      case 1024: RELAX_AMD_FUSED(true, 1024); break;
      case 512: RELAX_AMD_FUSED(true, 512); break;
      default: RELAX_AMD_FUSED(true, 256); break;
    }
  }
#undef RELAX_AMD_FUSED
  return check_launch("actor_step_fused");
}

}  // namespace relax_amd

using namespace relax_amd;

extern "C" int relax_amd_actor_step_fused(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                                          int64_t row_stride, const int32_t* token_of_row, const int32_t* sample_ids,
                                          const int64_t* targets, float inv_temperature,
                                          const relax_amd_policy_loss_args* loss, float grad_scale, float* log_prob,
                                          float* entropy, float* lse, float* spx, void* dlogits, int64_t d_row_stride,
                                          void* stream) {
  if (n_rows < 0 || n_rows > 2147483647LL || vocab <= 0 || row_stride < vocab || d_row_stride < vocab) {
    set_error("actor_step_fused: bad shape n_rows=%lld vocab=%lld", (long long)n_rows, (long long)vocab);
    return RELAX_AMD_EINVAL;
  }
  if (n_rows == 0) return RELAX_AMD_OK;
  if (loss && policy_loss_args_size_error(loss)) {
    set_error("actor_step_fused: %s", policy_loss_args_size_error(loss));
    return RELAX_AMD_EINVAL;
  }
  if (!logits || !targets || !loss || !log_prob || !entropy || !lse || !spx || !dlogits || !loss->advantages ||
      !loss->loss_mask || !loss->coef_log_prob) {
    set_error("actor_step_fused: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  const char* why = distill_args_error(*loss);
  if (!why) why = topk_distill_args_error(*loss);
  if (why) {
    set_error("actor_step_fused: %s", why);
    return RELAX_AMD_EINVAL;
  }
  if (!(inv_temperature > 0.f)) {
    set_error("actor_step_fused: inv_temperature must be > 0");
    return RELAX_AMD_EINVAL;
  }
  if (loss->loss_kind == RELAX_AMD_LOSS_GSPO || loss->use_opsm) {
    set_error("actor_step_fused: GSPO / OPSM couple the tokens of a sequence; use the two-launch path");
    return RELAX_AMD_EUNSUPPORTED;
  }
  if (loss->loss_kind < RELAX_AMD_LOSS_PPO || loss->loss_kind > RELAX_AMD_LOSS_SAPO ||
      loss->kl_kind < RELAX_AMD_KL_NONE || loss->kl_kind > RELAX_AMD_KL_LOW_VAR ||
      (loss->kl_kind != RELAX_AMD_KL_NONE && !loss->ref_log_prob)) {
    set_error("actor_step_fused: bad loss_kind / kl_kind or missing ref_log_prob");
    return RELAX_AMD_EINVAL;
  }
  if ((loss->sample_denom || loss->pg_sample_denom) && !sample_ids) {
    set_error("actor_step_fused: sample_ids is required with per-sample denominators");
    return RELAX_AMD_EINVAL;
  }
  if (dtype != RELAX_AMD_F32 && dtype != RELAX_AMD_BF16 && dtype != RELAX_AMD_F16) {
    set_error("actor_step_fused: unknown dtype code %d", dtype);
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32:
      return dispatch_fused<float>(logits, n_rows, vocab, row_stride, token_of_row, sample_ids, targets,
                                   inv_temperature, *loss, grad_scale, log_prob, entropy, lse, spx, dlogits,
                                   d_row_stride, s);
    case RELAX_AMD_BF16:
      return dispatch_fused<bf16_t>(logits, n_rows, vocab, row_stride, token_of_row, sample_ids, targets,
                                    inv_temperature, *loss, grad_scale, log_prob, entropy, lse, spx, dlogits,
                                    d_row_stride, s);
    default:
      return dispatch_fused<f16_t>(logits, n_rows, vocab, row_stride, token_of_row, sample_ids, targets,
                                   inv_temperature, *loss, grad_scale, log_prob, entropy, lse, spx, dlogits,
                                   d_row_stride, s);
  }
}

// dlogits *= (*factor) in place.  Skipped entirely (one compare per workgroup) when the factor is 1 to within 2^-20:
// the autograd backward of the fused step passes upstream / assumed here, and a chain of fp32 multiplications that
// mathematically equals the assumed scale may differ from it in the last bits; a relative 1e-6 is far below the
// rounding of the stored gradients.  Lets the backward honour an upstream gradient that differs from the scale
// assumed at forward time without a host read-back.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void rescale_rows_kernel(T* __restrict__ data, int64_t stride, int64_t vocab,
                                                           int64_t n_rows, const float* __restrict__ factor) {
  const float f = *factor;
  if (fabsf(f - 1.0f) <= 0x1p-20f) return;
  // a bounded grid walks the rows: in the usual case (factor 1) the launch is a few thousand workgroups that return
  // at once instead of one per row
  for (int64_t row = blockIdx.x; row < n_rows; row += gridDim.x) {
    T* r = data + row * stride;
    if constexpr (VEC) {
      constexpr int kPer = Row<T>::kPerVec;
      u32x4* rv = reinterpret_cast<u32x4*>(r);
      const int64_t nvec = vocab / kPer;
      for (int64_t i = threadIdx.x; i < nvec; i += 256) {
        float x[kPer];
        Row<T>::unpack(rv[i], x);
  #pragma unroll
        for (int k = 0; k < kPer; ++k) x[k] *= f;
        rv[i] = Row<T>::pack(x);
      }
      for (int64_t e = nvec * kPer + threadIdx.x; e < vocab; e += 256) Row<T>::store1(r + e, Row<T>::load1(r + e) * f);
    } else {
      for (int64_t e = threadIdx.x; e < vocab; e += 256) Row<T>::store1(r + e, Row<T>::load1(r + e) * f);
    }
  }
}

template <typename T>
static void launch_rescale(void* data, int64_t n_rows, int64_t vocab, int64_t stride, const float* factor,
                           hipStream_t s) {
  const bool vec = aligned16(data) && (stride * int64_t(sizeof(T))) % 16 == 0;
  const dim3 grid(static_cast<unsigned>(n_rows < 4096 ? n_rows : 4096)), block(256);
  if (vec)
    hipLaunchKernelGGL((rescale_rows_kernel<T, true>), grid, block, 0, s, static_cast<T*>(data), stride, vocab, n_rows,
                       factor);
  else
    hipLaunchKernelGGL((rescale_rows_kernel<T, false>), grid, block, 0, s, static_cast<T*>(data), stride, vocab, n_rows,
                       factor);
}

extern "C" int relax_amd_scale_rows_inplace(void* data, int dtype, int64_t n_rows, int64_t vocab, int64_t row_stride,
                                            const float* factor_dev, void* stream) {
  if (n_rows < 0 || n_rows > 2147483647LL || vocab <= 0 || row_stride < vocab || !data || !factor_dev) {
    set_error("scale_rows_inplace: bad arguments");
    return RELAX_AMD_EINVAL;
  }
  if (dtype != RELAX_AMD_F32 && dtype != RELAX_AMD_BF16 && dtype != RELAX_AMD_F16) {
    set_error("scale_rows_inplace: unknown dtype code %d", dtype);
    return RELAX_AMD_EINVAL;
  }
  if (n_rows == 0) return RELAX_AMD_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == RELAX_AMD_F32) launch_rescale<float>(data, n_rows, vocab, row_stride, factor_dev, s);
  else if (dtype == RELAX_AMD_BF16) launch_rescale<bf16_t>(data, n_rows, vocab, row_stride, factor_dev, s);
  else launch_rescale<f16_t>(data, n_rows, vocab, row_stride, factor_dev, s);
  return check_launch("rescale_rows");
}
