// Streaming log-prob + entropy forward and dlogits backward over [rows, vocab] logits.
//
// One workgroup owns one row.  The row is read once with 16-byte non-temporal loads (8 bf16 / 4 fp32 per lane
// per load, 4 loads in flight per lane); every lane keeps a private online-softmax state (running max, sum of
// exp, sum of exp * x) in the log2 domain so the inner loop is cvt + fma + v_exp_f32 + add + fma per element and the
// max rescale is paid once per 32 elements (row_scan.h).  Lane states are merged by a wave64 xor-butterfly, then
// across waves through LDS in wave order, so results are bit-identical run to run and identical to the forward
// half of the fused actor-step kernel.
//
// Arithmetic follows relax/utils/training/ppo_utils.py:481-629 (reference paths are relative to its checkout):
//   lp = x[tok] - lse,  H = lse - sum_v p*x,  dx = g_lp*(onehot - p) + g_H*p*(sum_v p*x - x),  x = logits / T.
#include <cstdlib>
#include <cstring>

#include "device_utils.h"
#include "logprob_bwd_resident.h"
#include "relax_amd.h"
#include "row_scan.h"

namespace relax_amd {

constexpr int kRowThreads = 256;  // backward kernel width
constexpr int kRowUnroll = 4;

// WITH_T = false: neither the entropy nor sum p*x is wanted (the forward-only pass of the ActorFwd / Reference roles,
// relax/backends/megatron/model.py:844 with use_rollout_entropy off): the scan drops that sum, log_prob and lse are
// the same bits.
template <typename T, bool VEC, int THREADS, bool WITH_T = true>
__global__ __launch_bounds__(THREADS) void logprob_entropy_fwd_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t vocab, const int32_t* __restrict__ row_ids,
    const int64_t* __restrict__ targets, float c, float inv_t, float* __restrict__ log_prob,
    float* __restrict__ entropy, float* __restrict__ lse_out, float* __restrict__ spx_out) {
  __shared__ float wave_state[THREADS / kWave][3];
  const int64_t tok = blockIdx.x;
  const int64_t row = row_ids ? int64_t(row_ids[tok]) : tok;
  const T* x = logits + row * row_stride;
  float x_target = 0.f;
  int64_t tg = -1;
  if (threadIdx.x == 0) {
    tg = targets[tok];
    if (tg >= 0 && tg < vocab) x_target = Row<T>::load1(x + tg);
  }
  SoftmaxAcc st = scan_row<T, VEC, true, THREADS, ScanNoHook, WITH_T>(x, vocab, c);
  scan_block_merge<THREADS>(st, wave_state);
  if (threadIdx.x == 0) {
    float lse, spx, ent, lp;
    scan_finish(st, x_target, tg >= 0 && tg < vocab, inv_t, lse, spx, ent, lp);
    log_prob[tok] = lp;
    if (WITH_T && entropy) entropy[tok] = ent;
    if (WITH_T && spx_out) spx_out[tok] = spx;
    if (lse_out) lse_out[tok] = lse;
  }
}

template <typename T, bool VEC>
__device__ __forceinline__ void zero_row(T* __restrict__ d, int64_t vocab) {
  if (VEC) {
    constexpr int VN = Row<T>::kPerVec;
    u32x4* dv = reinterpret_cast<u32x4*>(d);
    const int64_t nvec = vocab / VN;
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (int64_t i = threadIdx.x; i < nvec; i += kRowThreads) store_stream(dv + i, z);
    for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kRowThreads) Row<T>::store1(d + e, 0.f);
  } else {
    for (int64_t e = threadIdx.x; e < vocab; e += kRowThreads) Row<T>::store1(d + e, 0.f);
  }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kRowThreads) void logprob_entropy_bwd_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t vocab, const int32_t* __restrict__ token_of_row,
    const int64_t* __restrict__ targets, const float* __restrict__ lse, const float* __restrict__ spx,
    const float* __restrict__ g_lp, const float* __restrict__ g_ent, float grad_scale,
    const float* __restrict__ grad_scale_dev, float c, float inv_t,
    T* __restrict__ dlogits, int64_t d_stride) {
  const int64_t row = blockIdx.x;
  T* d = dlogits + row * d_stride;
  const int64_t tok = token_of_row ? int64_t(token_of_row[row]) : row;
  float glp = 0.f, gh = 0.f;
  if (tok >= 0) {
    if (grad_scale_dev) grad_scale *= *grad_scale_dev;
    glp = g_lp[tok] * grad_scale;
    gh = g_ent ? g_ent[tok] * grad_scale : 0.f;
  }
  if (tok < 0 || (glp == 0.f && gh == 0.f)) {
    zero_row<T, VEC>(d, vocab);
    return;
  }
  const T* x = logits + row * row_stride;
  const float k0 = -lse[tok] * kLog2e;  // p = exp2(x*c + k0)
  // d = inv_t * p * (-glp + gh * (spx - x*inv_t))  (+ inv_t*glp at the target)
  const float b = gh * inv_t;
  const float a0 = -glp * inv_t + (gh != 0.f ? b * spx[tok] : 0.f);
  const float a1 = -b * inv_t;
  const float hot = glp * inv_t;
  const int64_t tg = targets[tok];
  if (VEC) {
    constexpr int VN = Row<T>::kPerVec;
    const u32x4* xv = reinterpret_cast<const u32x4*>(x);
    u32x4* dv = reinterpret_cast<u32x4*>(d);
    const int64_t nvec = vocab / VN;
    const int64_t tvec = (tg >= 0 && tg < nvec * VN) ? tg / VN : -1;
    const int tsub = int(tg % VN);
    int64_t i = threadIdx.x;
    for (; i + int64_t(kRowUnroll - 1) * kRowThreads < nvec; i += int64_t(kRowUnroll) * kRowThreads) {
      u32x4 raw[kRowUnroll];
#pragma unroll
      for (int u = 0; u < kRowUnroll; ++u) raw[u] = load_stream(xv + i + int64_t(u) * kRowThreads);
#pragma unroll
      for (int u = 0; u < kRowUnroll; ++u) {
        float v[VN];
        Row<T>::unpack(raw[u], v);
#pragma unroll
        for (int k = 0; k < VN; ++k) v[k] = fast_exp2(fmaf(v[k], c, k0)) * fmaf(v[k], a1, a0);
        if (i + int64_t(u) * kRowThreads == tvec) {
#pragma unroll
          for (int k = 0; k < VN; ++k)
            if (k == tsub) v[k] += hot;
        }
        store_stream(dv + i + int64_t(u) * kRowThreads, Row<T>::pack(v));
      }
    }
    for (; i < nvec; i += kRowThreads) {
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
    for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kRowThreads) {
      const float xe = Row<T>::load1(x + e);
      float g = fast_exp2(fmaf(xe, c, k0)) * fmaf(xe, a1, a0);
      if (e == tg) g += hot;
      Row<T>::store1(d + e, g);
    }
  } else {
    for (int64_t e = threadIdx.x; e < vocab; e += kRowThreads) {
      const float xe = Row<T>::load1(x + e);
      float g = fast_exp2(fmaf(xe, c, k0)) * fmaf(xe, a1, a0);
      if (e == tg) g += hot;
      Row<T>::store1(d + e, g);
    }
  }
}

// The same backward in the form the memory system serves fastest when nothing has to stay on chip between a row's
// read and its write: workgroups of 256 threads that each take 4 KB of a row (one 16-byte vector per thread), in
// address order over rows and chunks, and exit.  At any moment the chip as a whole sweeps a short window of
// consecutive addresses instead of one row-sized stream per CU.  The row's coefficients come from uniform (scalar)
// loads; rows without gradient are written as zeros without a read.  Same arithmetic per element as the kernel above.
constexpr int kChunkThreads = 256;
template <typename T>
__global__ __launch_bounds__(kChunkThreads) void logprob_entropy_bwd_chunk_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t nvec, unsigned chunks_per_row,
    const int32_t* __restrict__ token_of_row, const int64_t* __restrict__ targets, const float* __restrict__ lse,
    const float* __restrict__ spx, const float* __restrict__ g_lp, const float* __restrict__ g_ent, float grad_scale,
    const float* __restrict__ grad_scale_dev, float c, float inv_t, T* __restrict__ dlogits, int64_t d_stride) {
  constexpr int VN = Row<T>::kPerVec;
  const unsigned b = blockIdx.x;
  const unsigned row = b / chunks_per_row, chunk = b - row * chunks_per_row;
  const int64_t i = int64_t(chunk) * kChunkThreads + threadIdx.x;
  if (i >= nvec) return;
  u32x4* dv = reinterpret_cast<u32x4*>(dlogits + int64_t(row) * d_stride);
  const int64_t tok = token_of_row ? int64_t(token_of_row[row]) : int64_t(row);
  float glp = 0.f, gh = 0.f;
  if (tok >= 0) {
    if (grad_scale_dev) grad_scale *= *grad_scale_dev;
    glp = g_lp[tok] * grad_scale;
    gh = g_ent ? g_ent[tok] * grad_scale : 0.f;
  }
  if (tok < 0 || (glp == 0.f && gh == 0.f)) {
    store_stream(dv + i, u32x4{0u, 0u, 0u, 0u});
    return;
  }
  const u32x4 raw = load_stream(reinterpret_cast<const u32x4*>(logits + int64_t(row) * row_stride) + i);
  const float k0 = -lse[tok] * kLog2e;
  const float bb = gh * inv_t;
  const float a0 = -glp * inv_t + (gh != 0.f ? bb * spx[tok] : 0.f);
  const float a1 = -bb * inv_t;
  const float hot = glp * inv_t;
  const int64_t tg = targets[tok];
  const int64_t tvec = (tg >= 0 && tg < nvec * VN) ? tg / VN : -1;
  const int tsub = int(tg % VN);
  float v[VN];
  Row<T>::unpack(raw, v);
#pragma unroll
  for (int k = 0; k < VN; ++k) v[k] = fast_exp2(fmaf(v[k], c, k0)) * fmaf(v[k], a1, a0);
  if (i == tvec) {
#pragma unroll
    for (int k = 0; k < VN; ++k)
      if (k == tsub) v[k] += hot;
  }
  store_stream(dv + i, Row<T>::pack(v));
}

template <typename T>
static int launch_fwd(const void* logits, int64_t n, int64_t vocab, int64_t stride, const int32_t* row_ids,
                      const int64_t* targets, float inv_t, float* lp, float* ent, float* lse, float* spx,
                      hipStream_t s) {
  const bool vec = aligned16(logits) && (stride * int64_t(sizeof(T))) % 16 == 0;
  const float c = inv_t * kLog2e;
  const T* x = static_cast<const T*>(logits);
  dim3 grid(static_cast<unsigned>(n));
  const bool with_t = ent || spx;  // neither asked for: the scan leaves sum p*x out
#define RELAX_AMD_FWD(V, TH)                                                                                        \
  if (with_t || !V)                                                                                                 \
    hipLaunchKernelGGL((logprob_entropy_fwd_kernel<T, V, TH, true>), grid, dim3(TH), 0, s, x, stride, vocab, row_ids, \
                       targets, c, inv_t, lp, ent, lse, spx);                                                       \
  else                                                                                                              \
    hipLaunchKernelGGL((logprob_entropy_fwd_kernel<T, V, TH, false>), grid, dim3(TH), 0, s, x, stride, vocab,       \
                       row_ids, targets, c, inv_t, lp, ent, lse, spx)
  if (!vec) {
    RELAX_AMD_FWD(false, 256);
  } else {
    switch (scan_threads(vocab, Row<T>::kPerVec)) {
      case 1024: RELAX_AMD_FWD(true, 1024); break;
      case 512: RELAX_AMD_FWD(true, 512); break;
      default: RELAX_AMD_FWD(true, 256); break;
    }
  }
#undef RELAX_AMD_FWD
  return check_launch("logprob_entropy_fwd");
}

template <typename T>
static int launch_bwd(const void* logits, int64_t n_rows, int64_t vocab, int64_t stride, const int32_t* token_of_row,
                      const int64_t* targets, const float* lse, const float* spx, const float* g_lp,
                      const float* g_ent, float grad_scale, const float* grad_scale_dev, float inv_t, void* dlogits,
                      int64_t d_stride, hipStream_t s) {
  const bool vec = aligned16(logits) && aligned16(dlogits) && (stride * int64_t(sizeof(T))) % 16 == 0 &&
                   (d_stride * int64_t(sizeof(T))) % 16 == 0;
  const float c = inv_t * kLog2e;
  dim3 grid(static_cast<unsigned>(n_rows)), block(kRowThreads);
  const T* x = static_cast<const T*>(logits);
  T* d = static_cast<T*>(dlogits);
  // Rows of whole 16-byte vectors take the chunk form (same bits, fastest).  relax_amd_set_kernel_choice: TWO_WALK
  // keeps every row length on the row-per-workgroup kernel; RESIDENT asks for the persistent burst form and fails
  // where it is not built (for tests that compare the forms).
  const int choice = kernel_choice();
  constexpr int VN = Row<T>::kPerVec;
  if (vec && choice == RELAX_AMD_KERNEL_AUTO && vocab % VN == 0) {
    const int64_t nvec = vocab / VN;
    const int64_t chunks = (nvec + kChunkThreads - 1) / kChunkThreads;
    if (n_rows * chunks <= 2147483647LL) {
      hipLaunchKernelGGL((logprob_entropy_bwd_chunk_kernel<T>), dim3(static_cast<unsigned>(n_rows * chunks)),
                         dim3(kChunkThreads), 0, s, x, stride, nvec, static_cast<unsigned>(chunks), token_of_row,
                         targets, lse, spx, g_lp, g_ent, grad_scale, grad_scale_dev, c, inv_t, d, d_stride);
      return check_launch("logprob_entropy_bwd_chunk");
    }
  }
  if (vec && choice != RELAX_AMD_KERNEL_TWO_WALK) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    const int rc = launch_logprob_bwd_resident<T>(x, stride, vocab, n_rows, token_of_row, targets, lse, spx, g_lp,
                                                  g_ent, grad_scale, grad_scale_dev, inv_t, d, d_stride, cus, s);
    if (rc != RELAX_AMD_EUNSUPPORTED) return rc;  // launched (or failed to): otherwise the row length is not built
  }
  if (choice == RELAX_AMD_KERNEL_RESIDENT) {
    set_error("logprob_entropy_bwd: kernel choice RESIDENT, but no burst-form kernel is built for rows "
              "of %lld elements of this type and alignment", (long long)vocab);
    return RELAX_AMD_EUNSUPPORTED;
  }
  if (vec)
    hipLaunchKernelGGL((logprob_entropy_bwd_kernel<T, true>), grid, block, 0, s, x, stride, vocab, token_of_row,
                       targets, lse, spx, g_lp, g_ent, grad_scale, grad_scale_dev, c, inv_t, d, d_stride);
  else
    hipLaunchKernelGGL((logprob_entropy_bwd_kernel<T, false>), grid, block, 0, s, x, stride, vocab, token_of_row,
                       targets, lse, spx, g_lp, g_ent, grad_scale, grad_scale_dev, c, inv_t, d, d_stride);
  return check_launch("logprob_entropy_bwd");
}

}  // namespace relax_amd

using namespace relax_amd;

static const int64_t kMaxGrid = 2147483647LL;

extern "C" int relax_amd_logprob_entropy_fwd(const void* logits, int dtype, int64_t n_tokens, int64_t vocab,
                                             int64_t row_stride, const int32_t* row_ids, const int64_t* targets,
                                             float inv_temperature, float* log_prob, float* entropy, float* lse,
                                             float* spx, void* stream) {
  if (n_tokens < 0 || n_tokens > kMaxGrid || vocab <= 0 || row_stride < vocab) {
    set_error("logprob_entropy_fwd: bad shape n_tokens=%lld vocab=%lld row_stride=%lld", (long long)n_tokens,
              (long long)vocab, (long long)row_stride);
    return RELAX_AMD_EINVAL;
  }
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (!logits || !targets || !log_prob) {
    set_error("logprob_entropy_fwd: logits, targets and log_prob must not be NULL");
    return RELAX_AMD_EINVAL;
  }
  if (!(inv_temperature > 0.f)) {
    set_error("logprob_entropy_fwd: inv_temperature must be > 0");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32:
      return launch_fwd<float>(logits, n_tokens, vocab, row_stride, row_ids, targets, inv_temperature, log_prob,
                               entropy, lse, spx, s);
    case RELAX_AMD_BF16:
      return launch_fwd<bf16_t>(logits, n_tokens, vocab, row_stride, row_ids, targets, inv_temperature, log_prob,
                                entropy, lse, spx, s);
    case RELAX_AMD_F16:
      return launch_fwd<f16_t>(logits, n_tokens, vocab, row_stride, row_ids, targets, inv_temperature, log_prob,
                               entropy, lse, spx, s);
    default:
      set_error("logprob_entropy_fwd: unknown dtype code %d", dtype);
      return RELAX_AMD_EINVAL;
  }
}

extern "C" int relax_amd_logprob_entropy_bwd(const void* logits, int dtype, int64_t n_rows, int64_t vocab,
                                             int64_t row_stride, const int32_t* token_of_row, const int64_t* targets,
                                             const float* lse, const float* spx, const float* g_lp,
                                             const float* g_ent, float grad_scale, const float* grad_scale_dev,
                                             float inv_temperature, void* dlogits, int64_t d_row_stride,
                                             void* stream) {
  if (n_rows < 0 || n_rows > kMaxGrid || vocab <= 0 || row_stride < vocab || d_row_stride < vocab) {
    set_error("logprob_entropy_bwd: bad shape n_rows=%lld vocab=%lld row_stride=%lld d_row_stride=%lld",
              (long long)n_rows, (long long)vocab, (long long)row_stride, (long long)d_row_stride);
    return RELAX_AMD_EINVAL;
  }
  if (n_rows == 0) return RELAX_AMD_OK;
  if (!logits || !targets || !lse || !g_lp || !dlogits || (g_ent && !spx)) {
    set_error("logprob_entropy_bwd: NULL argument (spx is required when g_ent is given)");
    return RELAX_AMD_EINVAL;
  }
  if (!(inv_temperature > 0.f)) {
    set_error("logprob_entropy_bwd: inv_temperature must be > 0");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32:
      return launch_bwd<float>(logits, n_rows, vocab, row_stride, token_of_row, targets, lse, spx, g_lp, g_ent,
                               grad_scale, grad_scale_dev, inv_temperature, dlogits, d_row_stride, s);
    case RELAX_AMD_BF16:
      return launch_bwd<bf16_t>(logits, n_rows, vocab, row_stride, token_of_row, targets, lse, spx, g_lp, g_ent,
                                grad_scale, grad_scale_dev, inv_temperature, dlogits, d_row_stride, s);
    case RELAX_AMD_F16:
      return launch_bwd<f16_t>(logits, n_rows, vocab, row_stride, token_of_row, targets, lse, spx, g_lp, g_ent,
                               grad_scale, grad_scale_dev, inv_temperature, dlogits, d_row_stride, s);
    default:
      set_error("logprob_entropy_bwd: unknown dtype code %d", dtype);
      return RELAX_AMD_EINVAL;
  }
}
