// Top-K on-policy distillation: log-probs of K given vocabulary ids per logits row, and the per-token KL family on
// [R, K] log-prob pairs with tail bin / renormalisation / truncation and the union path's padding mask.
//
//   topk_logprob_{fwd,bwd}  <- compute_log_probs_on_topk_token_ids   (relax/utils/opd/opd_utils.py:1022-1094)
//   opd_kl_topk_{fwd,bwd}   <- compute_opd_kl_topk / compute_opd_kl   (opd_utils.py:1097-1228)
//
// The gather is free once the row's log-sum-exp is known: the forward either reuses the lse the log-prob kernel
// already produced (K scalar loads per row) or scans the row itself; the backward is one streaming pass
// d[v] = -p[v] * sum_k g_k  followed by K read-modify-writes at the gathered positions.
#include "device_utils.h"
#include "opd_topk_math.h"
#include "relax_amd.h"
#include "row_scan.h"

namespace relax_amd {

constexpr int kTopkThreads = 256;

template <typename T, bool VEC>
__global__ __launch_bounds__(kTopkThreads) void topk_logprob_fwd_kernel(
    const T* __restrict__ logits, int64_t stride, int64_t vocab, const int32_t* __restrict__ row_ids,
    const int64_t* __restrict__ ids, int k_ids, float c, float inv_t, const float* __restrict__ lse_in,
    float* __restrict__ out, float* __restrict__ lse_out) {
  __shared__ float wave_state[kTopkThreads / kWave][3];
  __shared__ float bc_lse;
  const int64_t tok = blockIdx.x;
  const int64_t row = row_ids ? int64_t(row_ids[tok]) : tok;
  const T* x = logits + row * stride;
  float lse;
  if (lse_in) {
    lse = lse_in[tok];
  } else {
    SoftmaxAcc st = scan_row<T, VEC, true, kTopkThreads>(x, vocab, c);
    scan_block_merge<kTopkThreads>(st, wave_state);
    if (threadIdx.x == 0) {
      bc_lse = fmaf(st.m, kLn2, logf(st.s));
      if (lse_out) lse_out[tok] = bc_lse;
    }
    __syncthreads();
    lse = bc_lse;
  }
  for (int k = threadIdx.x; k < k_ids; k += kTopkThreads) {
    const int64_t id = ids[tok * k_ids + k];
    float v;
    if (id < 0)
      v = -INFINITY;  // sentinel
    else if (id >= vocab)
      v = -lse;  // outside the vocabulary slice: the reference gathers a zero logit
    else
      v = fmaf(Row<T>::load1(x + id), inv_t, -lse);
    out[tok * k_ids + k] = v;
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kTopkThreads) void topk_logprob_bwd_kernel(
    const T* __restrict__ logits, int64_t stride, int64_t vocab, const int32_t* __restrict__ token_of_row,
    const int64_t* __restrict__ ids, int k_ids, float c, float inv_t, const float* __restrict__ lse,
    const float* __restrict__ g, T* __restrict__ dlogits, int64_t d_stride) {
  __shared__ float part[kTopkThreads / kWave];
  const int64_t row = blockIdx.x;
  const int64_t tok = token_of_row ? int64_t(token_of_row[row]) : row;
  T* d = dlogits + row * d_stride;
  constexpr int VN = Row<T>::kPerVec;
  const int64_t nvec = VEC ? vocab / VN : 0;
  // G = sum of the incoming gradients of every non-sentinel id (each of them carries -lse)
  float gsum = 0.f;
  bool any = false;
  if (tok >= 0) {
    for (int k = threadIdx.x; k < k_ids; k += kTopkThreads) {
      const float gk = g[tok * k_ids + k];
      if (ids[tok * k_ids + k] >= 0 && gk != 0.f) {
        gsum += gk;
        any = true;
      }
    }
  }
  gsum = block_sum<kTopkThreads>(gsum, part);
  const bool live = __syncthreads_or(any);
  if (!live) {
    if (VEC) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (int64_t i = threadIdx.x; i < nvec; i += kTopkThreads) store_stream(reinterpret_cast<u32x4*>(d) + i, z);
    }
    for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kTopkThreads) Row<T>::store1(d + e, 0.f);
    return;
  }
  const T* x = logits + row * stride;
  const float k0 = -lse[tok] * kLog2e;
  const float a = -gsum * inv_t;
  if (VEC) {
    const u32x4* xv = reinterpret_cast<const u32x4*>(x);
    u32x4* dv = reinterpret_cast<u32x4*>(d);
    for (int64_t i = threadIdx.x; i < nvec; i += kTopkThreads) {
      float v[VN];
      Row<T>::unpack(load_stream(xv + i), v);
#pragma unroll
      for (int k = 0; k < VN; ++k) v[k] = fast_exp2(fmaf(v[k], c, k0)) * a;
      dv[i] = Row<T>::pack(v);  // ordinary store: a few entries of the row are patched right below
    }
  }
  for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kTopkThreads)
    Row<T>::store1(d + e, fast_exp2(fmaf(Row<T>::load1(x + e), c, k0)) * a);
  __threadfence_block();
  __syncthreads();
  if (threadIdx.x == 0) {  // sequential: repeated ids accumulate
    for (int k = 0; k < k_ids; ++k) {
      const int64_t id = ids[tok * k_ids + k];
      const float gk = g[tok * k_ids + k];
      if (id >= 0 && id < vocab && gk != 0.f) {
        T* slot = d + id;
        const float cur = Row<T>::load1(const_cast<const T*>(slot));
        Row<T>::store1(slot, fmaf(gk, inv_t, cur));
        __threadfence_block();
      }
    }
  }
}

// ---- per-token KL on [R, K] ------------------------------------------------------------------------------------

// One wave per row; the row's clamped + masked log-probs are staged in LDS (k is a run-time size).
template <bool BWD>
__global__ __launch_bounds__(256) void opd_kl_topk_kernel(const float* __restrict__ s_lp,
    const float* __restrict__ t_lp,
                                                          const uint8_t* __restrict__ mask, int64_t n_rows, int k_ids,
                                                          OpdParams p, const float* __restrict__ g,
                                                          float* __restrict__ out, float* __restrict__ d_s) {
  extern __shared__ float stage[];  // [4 waves][2][k_ids]
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  const int64_t r = blockIdx.x * 4LL + w;
  if (r >= n_rows) return;
  float* sv = stage + (w * 2) * k_ids;
  const float* s = s_lp + r * k_ids;
  const float* t = t_lp + r * k_ids;
  const uint8_t* mk = mask ? mask + r * k_ids : nullptr;
  const float gr = BWD ? g[r] : 0.f;
  const float acc = opd_kl_row<BWD>(
      k_ids, mk != nullptr, p, lane, sv, sv + k_ids, [&](int k) { return s[k]; }, [&](int k) { return t[k]; },
      [&](int k) { return mk[k] != 0; },
      [&](int k, float dk, bool nonzero) { d_s[r * k_ids + k] = nonzero ? gr * dk : 0.f; });
  if (!BWD && lane == 0) out[r] = acc;
}

// dlogits[row(t), id] += value * scale for the K (id, value) pairs of token t plus one pair at its target id: the
// sparse part of a gradient whose dense part (a multiple of the row's softmax) another kernel has already written.
// One thread walks all pairs of a token one after the other, so two pairs on the same element (a gathered id that
// equals the target) cannot race; ids outside [0, vocab) and tokens whose row id is negative are skipped.  (The form for very long lists; the usual ones
// take sparse_row_add_wave_kernel below.)
template <typename T>
__global__ __launch_bounds__(256) void sparse_row_add_kernel(T* __restrict__ dlogits, int64_t stride, int64_t vocab,
                                                             const int32_t* __restrict__ row_ids,
                                                             const int64_t* __restrict__ ids,
                                                             const float* __restrict__ values, int k,
                                                             const int64_t* __restrict__ targets,
                                                             const float* __restrict__ target_values, float scale,
                                                             int64_t n_tokens) {
  const int64_t tok = blockIdx.x * 256LL + threadIdx.x;
  if (tok >= n_tokens) return;
  const int64_t row = row_ids ? int64_t(row_ids[tok]) : tok;
  if (row < 0) return;  // a token without a row
  T* d = dlogits + row * stride;
  for (int j = 0; j < k; ++j) {
    const int64_t id = ids[tok * k + j];
    const float v = values[tok * k + j];
    if (id >= 0 && id < vocab && v != 0.f) Row<T>::store1(d + id, Row<T>::load1(d + id) + v * scale);
  }
  if (targets) {
    const int64_t id = targets[tok];
    const float v = target_values[tok];
    if (id >= 0 && id < vocab && v != 0.f) Row<T>::store1(d + id, Row<T>::load1(d + id) + v * scale);
  }
}

// The same for up to kSparseWaveMax pairs per token, one wave per token: lane l takes pairs l, l + 64, ... (the target
// pair counts as the last one).  Pairs on the same element are all applied by the lane of the first of them, so no two
// lanes touch one element; elements are read and written at their own width, so neighbours in one 32-bit word do not
// collide.
constexpr int kSparseWaveMax = 1024;

template <typename T>
__global__ __launch_bounds__(256) void sparse_row_add_wave_kernel(T* __restrict__ dlogits, int64_t stride,
                                                                  int64_t vocab, const int32_t* __restrict__ row_ids,
                                                                  const int64_t* __restrict__ ids,
                                                                  const float* __restrict__ values, int k,
                                                                  const int64_t* __restrict__ targets,
                                                                  const float* __restrict__ target_values, float scale,
                                                                  int64_t n_tokens) {
  extern __shared__ int64_t sparse_stage[];  // [4 waves][k + 1] ids, then [4 waves][k + 1] values
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  const int64_t tok = blockIdx.x * 4LL + w;
  if (tok >= n_tokens) return;
  const int64_t row = row_ids ? int64_t(row_ids[tok]) : tok;
  if (row < 0) return;  // a token without a row (uniform over the wave)
  const int n = k + (targets ? 1 : 0);
  int64_t* sid = sparse_stage + w * (k + 1);
  float* sval = reinterpret_cast<float*>(sparse_stage + 4 * (k + 1)) + w * (k + 1);
  for (int j = lane; j < n; j += kWave) {
    const int64_t id = j < k ? ids[tok * k + j] : targets[tok];
    const float v = j < k ? values[tok * k + j] : target_values[tok];
    const bool live = id >= 0 && id < vocab && v != 0.f;
    sid[j] = live ? id : -1;
    sval[j] = v;
  }
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  T* d = dlogits + row * stride;
  for (int j = lane; j < n; j += kWave) {
    const int64_t id = sid[j];
    if (id < 0) continue;
    bool first = true;
    for (int o = 0; o < j; ++o) first = first && sid[o] != id;
    if (!first) continue;
    // this pair and, one after the other, the later ones on the same element: each addition rounded to the element
    // type, as a walk over the list in its order would do
    T* slot = d + id;
    Row<T>::store1(slot, Row<T>::load1(const_cast<const T*>(slot)) + sval[j] * scale);
    for (int o = j + 1; o < n; ++o)
      if (sid[o] == id) Row<T>::store1(slot, Row<T>::load1(const_cast<const T*>(slot)) + sval[o] * scale);
  }
}

}  // namespace relax_amd

using namespace relax_amd;

extern "C" int relax_amd_sparse_row_add(void* dlogits, int dtype, int64_t n_tokens, int64_t vocab, int64_t row_stride,
                                        const int32_t* row_ids, const int64_t* ids, const float* values, int64_t k,
                                        const int64_t* targets, const float* target_values, float scale,
                                        void* stream) {
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (n_tokens < 0 || n_tokens > 2147483647LL || vocab <= 0 || row_stride < vocab || k < 0 || k > (1 << 20) ||
      !dlogits ||
      (k > 0 && (!ids || !values)) || (targets && !target_values)) {
    set_error("sparse_row_add: NULL argument or bad shape n=%lld vocab=%lld row_stride=%lld k=%lld",
              (long long)n_tokens, (long long)vocab, (long long)row_stride, (long long)k);
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (k < kSparseWaveMax) {  // one wave per token
    const dim3 wgrid(static_cast<unsigned>((n_tokens + 3) / 4)), wblock(256);
    const size_t lds = size_t(4) * size_t(k + 1) * (sizeof(int64_t) + sizeof(float));
#define RELAX_AMD_SPARSE_WAVE(T)                                                                                   \
  hipLaunchKernelGGL(sparse_row_add_wave_kernel<T>, wgrid, wblock, lds, s, static_cast<T*>(dlogits), row_stride,    \
                     vocab, row_ids, ids, values, int(k), targets, target_values, scale, n_tokens)
    switch (dtype) {
      case RELAX_AMD_F32: RELAX_AMD_SPARSE_WAVE(float); break;
      case RELAX_AMD_BF16: RELAX_AMD_SPARSE_WAVE(bf16_t); break;
      case RELAX_AMD_F16: RELAX_AMD_SPARSE_WAVE(f16_t); break;
      default: set_error("sparse_row_add: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
    }
#undef RELAX_AMD_SPARSE_WAVE
    return check_launch("sparse_row_add");
  }
  const dim3 grid(static_cast<unsigned>((n_tokens + 255) / 256)), block(256);
  switch (dtype) {
    case RELAX_AMD_F32:
      hipLaunchKernelGGL(sparse_row_add_kernel<float>, grid, block, 0, s, static_cast<float*>(dlogits), row_stride,
                         vocab, row_ids, ids, values, int(k), targets, target_values, scale, n_tokens);
      break;
    case RELAX_AMD_BF16:
      hipLaunchKernelGGL(sparse_row_add_kernel<bf16_t>, grid, block, 0, s, static_cast<bf16_t*>(dlogits), row_stride,
                         vocab, row_ids, ids, values, int(k), targets, target_values, scale, n_tokens);
      break;
    case RELAX_AMD_F16:
      hipLaunchKernelGGL(sparse_row_add_kernel<f16_t>, grid, block, 0, s, static_cast<f16_t*>(dlogits), row_stride,
                         vocab, row_ids, ids, values, int(k), targets, target_values, scale, n_tokens);
      break;
    default: set_error("sparse_row_add: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
  return check_launch("sparse_row_add");
}

static int topk_check(const char* what, int64_t n, int64_t vocab, int64_t stride, int64_t k) {
  if (n < 0 || n > 2147483647LL || vocab <= 0 || stride < vocab || k < 0 || k > (1 << 20)) {
    set_error("%s: bad shape n=%lld vocab=%lld row_stride=%lld k=%lld", what, (long long)n, (long long)vocab,
              (long long)stride, (long long)k);
    return RELAX_AMD_EINVAL;
  }
  return RELAX_AMD_OK;
}

template <typename T>
static int launch_topk_fwd(const void* logits, int64_t n, int64_t vocab, int64_t stride, const int32_t* row_ids,
                           const int64_t* ids, int k, float inv_t, const float* lse_in, float* out, float* lse_out,
                           hipStream_t s) {
  const bool vec = aligned16(logits) && (stride * int64_t(sizeof(T))) % 16 == 0;
  dim3 grid(static_cast<unsigned>(n)), block(kTopkThreads);
  if (vec)
    hipLaunchKernelGGL((topk_logprob_fwd_kernel<T, true>), grid, block, 0, s, static_cast<const T*>(logits), stride,
                       vocab, row_ids, ids, k, inv_t * kLog2e, inv_t, lse_in, out, lse_out);
  else
    hipLaunchKernelGGL((topk_logprob_fwd_kernel<T, false>), grid, block, 0, s, static_cast<const T*>(logits), stride,
                       vocab, row_ids, ids, k, inv_t * kLog2e, inv_t, lse_in, out, lse_out);
  return check_launch("topk_logprob_fwd");
}

template <typename T>
static int launch_topk_bwd(const void* logits, int64_t rows, int64_t vocab, int64_t stride,
                           const int32_t* token_of_row, const int64_t* ids, int k, float inv_t, const float* lse,
                           const float* g, void* d, int64_t d_stride, hipStream_t s) {
  const bool vec = aligned16(logits) && aligned16(d) && (stride * int64_t(sizeof(T))) % 16 == 0 &&
                   (d_stride * int64_t(sizeof(T))) % 16 == 0;
  dim3 grid(static_cast<unsigned>(rows)), block(kTopkThreads);
  if (vec)
    hipLaunchKernelGGL((topk_logprob_bwd_kernel<T, true>), grid, block, 0, s, static_cast<const T*>(logits), stride,
                       vocab, token_of_row, ids, k, inv_t * kLog2e, inv_t, lse, g, static_cast<T*>(d), d_stride);
  else
    hipLaunchKernelGGL((topk_logprob_bwd_kernel<T, false>), grid, block, 0, s, static_cast<const T*>(logits), stride,
                       vocab, token_of_row, ids, k, inv_t * kLog2e, inv_t, lse, g, static_cast<T*>(d), d_stride);
  return check_launch("topk_logprob_bwd");
}

extern "C" int relax_amd_topk_logprob_fwd(const void* logits, int dtype, int64_t n_tokens, int64_t vocab,
                                          int64_t row_stride, const int32_t* row_ids, const int64_t* topk_ids,
                                          int64_t k, float inv_temperature, const float* lse_in, float* topk_log_prob,
                                          float* lse_out, void* stream) {
  if (int rc = topk_check("topk_logprob_fwd", n_tokens, vocab, row_stride, k)) return rc;
  if (n_tokens == 0 || k == 0) return RELAX_AMD_OK;
  if (!logits || !topk_ids || !topk_log_prob || !(inv_temperature > 0.f)) {
    set_error("topk_logprob_fwd: NULL argument or non-positive inv_temperature");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32:
      return launch_topk_fwd<float>(logits, n_tokens, vocab, row_stride, row_ids, topk_ids, int(k), inv_temperature,
          lse_in, topk_log_prob, lse_out, s);
    case RELAX_AMD_BF16:
      return launch_topk_fwd<bf16_t>(logits, n_tokens, vocab, row_stride, row_ids, topk_ids, int(k), inv_temperature,
          lse_in, topk_log_prob, lse_out, s);
    case RELAX_AMD_F16:
      return launch_topk_fwd<f16_t>(logits, n_tokens, vocab, row_stride, row_ids, topk_ids, int(k), inv_temperature,
          lse_in, topk_log_prob, lse_out, s);
    default: set_error("topk_logprob_fwd: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
}

extern "C" int relax_amd_topk_logprob_bwd(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                                          int64_t row_stride, const int32_t* token_of_row, const int64_t* topk_ids,
                                          int64_t k, float inv_temperature, const float* lse, const float* g,
                                          void* dlogits, int64_t d_stride, void* stream) {
  if (int rc = topk_check("topk_logprob_bwd", n_rows, vocab, row_stride, k)) return rc;
  if (n_rows == 0) return RELAX_AMD_OK;
  if (!logits || !topk_ids || !lse || !g || !dlogits || d_stride < vocab || !(inv_temperature > 0.f)) {
    set_error("topk_logprob_bwd: NULL argument, short d_stride or non-positive inv_temperature");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32:
      return launch_topk_bwd<float>(logits, n_rows, vocab, row_stride, token_of_row, topk_ids, int(k),
          inv_temperature, lse, g, dlogits, d_stride, s);
    case RELAX_AMD_BF16:
      return launch_topk_bwd<bf16_t>(logits, n_rows, vocab, row_stride, token_of_row, topk_ids, int(k),
          inv_temperature, lse, g, dlogits, d_stride, s);
    case RELAX_AMD_F16:
      return launch_topk_bwd<f16_t>(logits, n_rows, vocab, row_stride, token_of_row, topk_ids, int(k),
          inv_temperature, lse, g, dlogits, d_stride, s);
    default: set_error("topk_logprob_bwd: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
}

static int opd_params(const char* what, int kl_mode, int norm_mode, float alpha, int has_clamp, float clamp,
                      int64_t n, int64_t k, OpdParams& p) {
  if (n < 0 || k <= 0 || k > 2048) {
    set_error("%s: bad shape n_rows=%lld k=%lld (k must be in 1..2048)", what, (long long)n, (long long)k);
    return RELAX_AMD_EINVAL;
  }
  if ((kl_mode != RELAX_AMD_OPD_JSD && kl_mode != RELAX_AMD_OPD_LOW_VAR) || norm_mode < RELAX_AMD_OPD_NORM_TAIL ||
      norm_mode > RELAX_AMD_OPD_NORM_TRUNC || !(alpha >= 0.f && alpha <= 1.f)) {
    set_error("%s: unknown kl mode %d / norm mode %d, or jsd_alpha %g outside [0, 1]", what, kl_mode, norm_mode,
              double(alpha));
    return RELAX_AMD_EINVAL;
  }
  p = OpdParams{kl_mode, norm_mode, alpha, has_clamp, clamp};
  return RELAX_AMD_OK;
}

extern "C" int relax_amd_opd_kl_topk_fwd(const float* student_lp, const float* teacher_lp, const uint8_t* mask,
                                         int64_t n_rows, int64_t k, int kl_mode, int norm_mode, float jsd_alpha,
                                         int has_clamp, float log_prob_min_clamp, float* kl, void* stream) {
  OpdParams p;
  if (int rc = opd_params("opd_kl_topk_fwd", kl_mode, norm_mode, jsd_alpha, has_clamp, log_prob_min_clamp, n_rows, k,
      p))
    return rc;
  if (n_rows == 0) return RELAX_AMD_OK;
  if (!student_lp || !teacher_lp || !kl) {
    set_error("opd_kl_topk_fwd: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  const size_t lds = size_t(4) * 2 * size_t(k) * sizeof(float);
  hipLaunchKernelGGL((opd_kl_topk_kernel<false>), dim3(unsigned((n_rows + 3) / 4)), dim3(256), lds,
                     static_cast<hipStream_t>(stream), student_lp, teacher_lp, mask, n_rows, int(k), p, nullptr, kl,
                     nullptr);
  return check_launch("opd_kl_topk_fwd");
}

extern "C" int relax_amd_opd_kl_topk_bwd(const float* student_lp, const float* teacher_lp, const uint8_t* mask,
                                         int64_t n_rows, int64_t k, int kl_mode, int norm_mode, float jsd_alpha,
                                         int has_clamp, float log_prob_min_clamp, const float* g, float* d_student_lp,
                                         void* stream) {
  OpdParams p;
  if (int rc = opd_params("opd_kl_topk_bwd", kl_mode, norm_mode, jsd_alpha, has_clamp, log_prob_min_clamp, n_rows, k,
      p))
    return rc;
  if (n_rows == 0) return RELAX_AMD_OK;
  if (!student_lp || !teacher_lp || !g || !d_student_lp) {
    set_error("opd_kl_topk_bwd: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  const size_t lds = size_t(4) * 2 * size_t(k) * sizeof(float);
  hipLaunchKernelGGL((opd_kl_topk_kernel<true>), dim3(unsigned((n_rows + 3) / 4)), dim3(256), lds,
                     static_cast<hipStream_t>(stream), student_lp, teacher_lp, mask, n_rows, int(k), p, g, nullptr,
                     d_student_lp);
  return check_launch("opd_kl_topk_bwd");
}
