// Log-prob + entropy with a per-entry vocabulary keep mask: the log-prob's softmax runs over the kept entries (and
// always the target), the entropy over the whole row.  log_prob_keep_mask branch of
// _VocabParallelLogProbEntropy.forward / .backward (relax/utils/training/ppo_utils.py:546-567, 597-629).
//
// One workgroup per row, one pass: each lane keeps two online-softmax states, the full one (max, sum e, sum e*x) and
// the kept one (masked-out entries enter as -huge and contribute exp2(-huge) = 0).  The mask costs one extra byte per
// vocabulary entry on top of the row itself.
#include "device_utils.h"
#include "relax_amd.h"
#include "row_scan.h"

namespace relax_amd {

constexpr int kMaskThreads = 256;

template <typename T, bool VEC>
__global__ __launch_bounds__(kMaskThreads) void logprob_entropy_masked_fwd_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t vocab, const int32_t* __restrict__ row_ids,
    const int64_t* __restrict__ targets, const uint8_t* __restrict__ keep, int64_t keep_stride, float c, float inv_t,
    float* __restrict__ log_prob, float* __restrict__ entropy, float* __restrict__ lse_kept,
    float* __restrict__ lse_full, float* __restrict__ spx_out) {
  __shared__ float ws_full[kMaskThreads / kWave][3];
  __shared__ float ws_kept[kMaskThreads / kWave][3];
  const int64_t tok = blockIdx.x;
  const int64_t row = row_ids ? int64_t(row_ids[tok]) : tok;
  const T* x = logits + row * row_stride;
  const uint8_t* mk = keep + tok * keep_stride;
  constexpr int VN = Row<T>::kPerVec;
  const int64_t nvec = VEC ? vocab / VN : 0;
  SoftmaxAcc full{kNegHuge, 0.f, 0.f}, kept{kNegHuge, 0.f, 0.f};
  if (VEC) {
    const u32x4* xv = reinterpret_cast<const u32x4*>(x);
    for (int64_t i = threadIdx.x; i < nvec; i += kMaskThreads) {
      float v[VN], vk[VN];
      Row<T>::unpack(load_stream(xv + i), v);
      uint8_t m[VN];
      if (VN == 8) {
        const uint64_t bits = *reinterpret_cast<const uint64_t*>(mk + i * VN);
#pragma unroll
        for (int k = 0; k < VN; ++k) m[k] = uint8_t(bits >> (8 * k));
      } else {
        const uint32_t bits = *reinterpret_cast<const uint32_t*>(mk + i * VN);
#pragma unroll
        for (int k = 0; k < VN; ++k) m[k] = uint8_t(bits >> (8 * k));
      }
#pragma unroll
      for (int k = 0; k < VN; ++k) vk[k] = m[k] ? v[k] : kNegHuge;
      scan_absorb(v, c, full);
      scan_absorb(vk, c, kept);
    }
  }
  for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kMaskThreads) {
    float v[1] = {Row<T>::load1(x + e)};
    float vk[1] = {mk[e] ? v[0] : kNegHuge};
    scan_absorb(v, c, full);
    scan_absorb(vk, c, kept);
  }
  scan_block_merge<kMaskThreads>(full, ws_full);
  scan_block_merge<kMaskThreads>(kept, ws_kept);
  if (threadIdx.x == 0) {
    const int64_t tg = targets[tok];
    const bool ok = tg >= 0 && tg < vocab;
    const float xt = ok ? Row<T>::load1(x + tg) : 0.f;
    if (ok && !mk[tg]) scan_merge(kept, xt * c, 1.f, xt);  // the target always takes part in its own softmax
    float lse, spx, ent, lp_full;
    scan_finish(full, xt, ok, inv_t, lse, spx, ent, lp_full);
    const float lk = fmaf(kept.m, kLn2, logf(kept.s));
    log_prob[tok] = ok ? fmaf(xt, inv_t, -lk) : __builtin_nanf("");
    lse_kept[tok] = lk;
    if (entropy) entropy[tok] = ent;
    if (lse_full) lse_full[tok] = lse;
    if (spx_out) spx_out[tok] = spx;
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kMaskThreads) void logprob_entropy_masked_bwd_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t vocab, const int32_t* __restrict__ token_of_row,
    const int64_t* __restrict__ targets, const uint8_t* __restrict__ keep, int64_t keep_stride,
    const float* __restrict__ lse_kept, const float* __restrict__ lse_full, const float* __restrict__ spx,
    const float* __restrict__ g_lp, const float* __restrict__ g_ent, float grad_scale, float c, float inv_t,
    T* __restrict__ dlogits, int64_t d_stride) {
  const int64_t row = blockIdx.x;
  T* d = dlogits + row * d_stride;
  const int64_t tok = token_of_row ? int64_t(token_of_row[row]) : row;
  constexpr int VN = Row<T>::kPerVec;
  const int64_t nvec = VEC ? vocab / VN : 0;
  float glp = 0.f, gh = 0.f;
  if (tok >= 0) {
    glp = g_lp[tok] * grad_scale;
    gh = g_ent ? g_ent[tok] * grad_scale : 0.f;
  }
  if (tok < 0 || (glp == 0.f && gh == 0.f)) {
    if (VEC) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (int64_t i = threadIdx.x; i < nvec; i += kMaskThreads) store_stream(reinterpret_cast<u32x4*>(d) + i, z);
    }
    for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kMaskThreads) Row<T>::store1(d + e, 0.f);
    return;
  }
  const T* x = logits + row * row_stride;
  const uint8_t* mk = keep + tok * keep_stride;
  const int64_t tg = targets[tok];
  const float kk = -lse_kept[tok] * kLog2e, kf = gh != 0.f ? -lse_full[tok] * kLog2e : 0.f;
  const float b = gh * inv_t;
  const float ak = -glp * inv_t;                 // kept softmax:  d += ak * p_kept
  const float a0 = gh != 0.f ? b * spx[tok] : 0.f;  // full softmax:  d += p_full * (a0 + a1 * x)
  const float a1 = -b * inv_t;
  const float hot = glp * inv_t;
  auto grad = [&](float xv, bool kept_entry, bool is_target) {
    float g = 0.f;
    if (kept_entry || is_target) g = ak * fast_exp2(fmaf(xv, c, kk));
    if (gh != 0.f) g = fmaf(fast_exp2(fmaf(xv, c, kf)), fmaf(xv, a1, a0), g);
    if (is_target) g += hot;
    return g;
  };
  if (VEC) {
    const u32x4* xv = reinterpret_cast<const u32x4*>(x);
    u32x4* dv = reinterpret_cast<u32x4*>(d);
    for (int64_t i = threadIdx.x; i < nvec; i += kMaskThreads) {
      float v[VN];
      Row<T>::unpack(load_stream(xv + i), v);
#pragma unroll
      for (int k = 0; k < VN; ++k) v[k] = grad(v[k], mk[i * VN + k] != 0, i * VN + k == tg);
      store_stream(dv + i, Row<T>::pack(v));
    }
  }
  for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kMaskThreads)
    Row<T>::store1(d + e, grad(Row<T>::load1(x + e), mk[e] != 0, e == tg));
}

template <typename T>
static int launch_masked_fwd(const void* logits, int64_t n, int64_t vocab, int64_t stride, const int32_t* row_ids,
                             const int64_t* targets, const uint8_t* keep, int64_t keep_stride, float inv_t, float* lp,
                             float* ent, float* lk, float* lf, float* spx, hipStream_t s) {
  const bool vec = aligned16(logits) && (stride * int64_t(sizeof(T))) % 16 == 0 &&
                   (reinterpret_cast<uintptr_t>(keep) & 7u) == 0 && keep_stride % 8 == 0;
  dim3 grid(static_cast<unsigned>(n)), block(kMaskThreads);
  if (vec)
    hipLaunchKernelGGL((logprob_entropy_masked_fwd_kernel<T, true>), grid, block, 0, s, static_cast<const T*>(logits),
                       stride, vocab, row_ids, targets, keep, keep_stride, inv_t * kLog2e, inv_t, lp, ent, lk, lf, spx);
  else
    hipLaunchKernelGGL((logprob_entropy_masked_fwd_kernel<T, false>), grid, block, 0, s, static_cast<const T*>(logits),
                       stride, vocab, row_ids, targets, keep, keep_stride, inv_t * kLog2e, inv_t, lp, ent, lk, lf, spx);
  return check_launch("logprob_entropy_masked_fwd");
}

template <typename T>
static int launch_masked_bwd(const void* logits, int64_t rows, int64_t vocab, int64_t stride,
                             const int32_t* token_of_row, const int64_t* targets, const uint8_t* keep,
                             int64_t keep_stride, const float* lk, const float* lf, const float* spx,
                             const float* g_lp, const float* g_ent, float scale, float inv_t, void* d,
                             int64_t d_stride, hipStream_t s) {
  const bool vec = aligned16(logits) && aligned16(d) && (stride * int64_t(sizeof(T))) % 16 == 0 &&
                   (d_stride * int64_t(sizeof(T))) % 16 == 0;
  dim3 grid(static_cast<unsigned>(rows)), block(kMaskThreads);
  if (vec)
    hipLaunchKernelGGL((logprob_entropy_masked_bwd_kernel<T, true>), grid, block, 0, s, static_cast<const T*>(logits),
                       stride, vocab, token_of_row, targets, keep, keep_stride, lk, lf, spx, g_lp, g_ent, scale,
                       inv_t * kLog2e, inv_t, static_cast<T*>(d), d_stride);
  else
    hipLaunchKernelGGL((logprob_entropy_masked_bwd_kernel<T, false>), grid, block, 0, s, static_cast<const T*>(logits),
                       stride, vocab, token_of_row, targets, keep, keep_stride, lk, lf, spx, g_lp, g_ent, scale,
                       inv_t * kLog2e, inv_t, static_cast<T*>(d), d_stride);
  return check_launch("logprob_entropy_masked_bwd");
}

}  // namespace relax_amd

using namespace relax_amd;

static int masked_check(const char* what, int64_t n, int64_t vocab, int64_t stride, int64_t keep_stride, float inv_t) {
  if (n < 0 || n > 2147483647LL || vocab <= 0 || stride < vocab || keep_stride < vocab) {
    set_error("%s: bad shape n=%lld vocab=%lld row_stride=%lld keep_stride=%lld", what, (long long)n,
              (long long)vocab, (long long)stride, (long long)keep_stride);
    return RELAX_AMD_EINVAL;
  }
  if (!(inv_t > 0.f)) {
    set_error("%s: inv_temperature must be > 0", what);
    return RELAX_AMD_EINVAL;
  }
  return RELAX_AMD_OK;
}

extern "C" int relax_amd_logprob_entropy_masked_fwd(const void* logits, int dtype, int64_t n_tokens, int64_t vocab,
                                                    int64_t row_stride, const int32_t* row_ids,
                                                    const int64_t* targets, const uint8_t* keep_mask,
                                                    int64_t keep_stride, float inv_temperature, float* log_prob,
                                                    float* entropy, float* lse_kept, float* lse_full, float* spx,
                                                    void* stream) {
  if (int rc = masked_check("logprob_entropy_masked_fwd", n_tokens, vocab, row_stride, keep_stride, inv_temperature))
    return rc;
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (!logits || !targets || !keep_mask || !log_prob || !lse_kept) {
    set_error("logprob_entropy_masked_fwd: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32:
      return launch_masked_fwd<float>(logits, n_tokens, vocab, row_stride, row_ids, targets, keep_mask, keep_stride,
          inv_temperature, log_prob, entropy, lse_kept, lse_full, spx, s);
    case RELAX_AMD_BF16:
      return launch_masked_fwd<bf16_t>(logits, n_tokens, vocab, row_stride, row_ids, targets, keep_mask, keep_stride,
          inv_temperature, log_prob, entropy, lse_kept, lse_full, spx, s);
    case RELAX_AMD_F16:
      return launch_masked_fwd<f16_t>(logits, n_tokens, vocab, row_stride, row_ids, targets, keep_mask, keep_stride,
          inv_temperature, log_prob, entropy, lse_kept, lse_full, spx, s);
    default: set_error("logprob_entropy_masked_fwd: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
}

extern "C" int relax_amd_logprob_entropy_masked_bwd(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                                                    int64_t row_stride, const int32_t* token_of_row,
                                                    const int64_t* targets, const uint8_t* keep_mask,
                                                    int64_t keep_stride, const float* lse_kept, const float* lse_full,
                                                    const float* spx, const float* g_lp, const float* g_ent,
                                                    float grad_scale, float inv_temperature, void* dlogits,
                                                    int64_t d_row_stride, void* stream) {
  if (int rc = masked_check("logprob_entropy_masked_bwd", n_rows, vocab, row_stride, keep_stride, inv_temperature))
    return rc;
  if (n_rows == 0) return RELAX_AMD_OK;
  if (!logits || !targets || !keep_mask || !lse_kept || !g_lp || !dlogits || d_row_stride < vocab ||
      (g_ent && (!spx || !lse_full))) {
    set_error("logprob_entropy_masked_bwd: NULL argument or short d_row_stride (spx and lse_full are required when "
              "g_ent is given)");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32:
      return launch_masked_bwd<float>(logits, n_rows, vocab, row_stride, token_of_row, targets, keep_mask,
          keep_stride, lse_kept, lse_full, spx, g_lp, g_ent, grad_scale, inv_temperature, dlogits, d_row_stride, s);
    case RELAX_AMD_BF16:
      return launch_masked_bwd<bf16_t>(logits, n_rows, vocab, row_stride, token_of_row, targets, keep_mask,
          keep_stride, lse_kept, lse_full, spx, g_lp, g_ent, grad_scale, inv_temperature, dlogits, d_row_stride, s);
    case RELAX_AMD_F16:
      return launch_masked_bwd<f16_t>(logits, n_rows, vocab, row_stride, token_of_row, targets, keep_mask,
          keep_stride, lse_kept, lse_full, spx, g_lp, g_ent, grad_scale, inv_temperature, dlogits, d_row_stride, s);
    default: set_error("logprob_entropy_masked_bwd: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
}
