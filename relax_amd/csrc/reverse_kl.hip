// Full-vocab reverse KL(student || teacher) per token and its gradient w.r.t. the student logits.
//
// Forward: one workgroup per token streams the student row and the teacher row together (16-byte non-temporal
// loads) and keeps two online-softmax states per lane:  (m_s, sum e_s, sum e_s*(x_s - x_t))  and  (m_t, sum e_t).
//   KL = sum_v p_s*(log p_s - log p_t) = sum_v p_s*(x_s - x_t) - lse_s + lse_t
// which is what the jsd_alpha == 0 branch of compute_opd_kl (relax/utils/opd/opd_utils.py:1165-1169) evaluates when
// its [R, K] inputs are complete log-softmax rows (K = vocab; the tail bin then carries zero mass).
// Backward: d KL / d x_s[v] = p_s[v] * ((log p_s[v] - log p_t[v]) - KL); reads both rows once, writes one.
#include "device_utils.h"
#include "relax_amd.h"
#include "reverse_kl_math.h"
#include "reverse_kl_resident.h"

#include <cstdlib>
#include <cstring>

namespace relax_amd {

template <typename T, bool VEC>
__global__ __launch_bounds__(kKlThreads) void reverse_kl_fwd_kernel(const T* __restrict__ student,
                                                                    const T* __restrict__ teacher, int64_t stride,
                                                                    int64_t vocab, float* __restrict__ kl,
                                                                    float* __restrict__ lse_s,
                                                                    float* __restrict__ lse_t) {
  __shared__ float lds[kKlThreads / kWave][5];
  const int64_t tok = blockIdx.x;
  const T* xs = student + tok * stride;
  const T* xt = teacher + tok * stride;
  KlState q{kNegHuge, 0.f, 0.f, kNegHuge, 0.f};
  if (VEC) {
    constexpr int VN = Row<T>::kPerVec;
    const u32x4* sv = reinterpret_cast<const u32x4*>(xs);
    const u32x4* tv = reinterpret_cast<const u32x4*>(xt);
    const int64_t nvec = vocab / VN;
    int64_t i = threadIdx.x;
    for (; i + int64_t(kKlUnroll - 1) * kKlThreads < nvec; i += int64_t(kKlUnroll) * kKlThreads) {
      u32x4 rs[kKlUnroll], rt[kKlUnroll];
#pragma unroll
      for (int u = 0; u < kKlUnroll; ++u) {
        rs[u] = load_stream(sv + i + int64_t(u) * kKlThreads);
        rt[u] = load_stream(tv + i + int64_t(u) * kKlThreads);
      }
      float a[kKlUnroll * VN], b[kKlUnroll * VN];
#pragma unroll
      for (int u = 0; u < kKlUnroll; ++u) {
        float pa[VN], pb[VN];
        Row<T>::unpack(rs[u], pa);
        Row<T>::unpack(rt[u], pb);
#pragma unroll
        for (int k = 0; k < VN; ++k) {
          a[u * VN + k] = pa[k];
          b[u * VN + k] = pb[k];
        }
      }
      absorb_pair(a, b, q);
    }
    for (; i < nvec; i += kKlThreads) {
      float a[VN], b[VN];
      Row<T>::unpack(load_stream(sv + i), a);
      Row<T>::unpack(load_stream(tv + i), b);
      absorb_pair(a, b, q);
    }
    for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kKlThreads) {
      float a[1] = {Row<T>::load1(xs + e)}, b[1] = {Row<T>::load1(xt + e)};
      absorb_pair(a, b, q);
    }
  } else {
    for (int64_t e = threadIdx.x; e < vocab; e += kKlThreads) {
      float a[1] = {Row<T>::load1(xs + e)}, b[1] = {Row<T>::load1(xt + e)};
      absorb_pair(a, b, q);
    }
  }
  wave_butterfly([&](auto o) {
    constexpr int O = decltype(o)::value;
    KlState other{lane_xor<O>(q.ms), lane_xor<O>(q.ss), lane_xor<O>(q.us), lane_xor<O>(q.mt), lane_xor<O>(q.st)};
    merge_kl(q, other);
  });
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  if (lane == 0) {
    lds[w][0] = q.ms;
    lds[w][1] = q.ss;
    lds[w][2] = q.us;
    lds[w][3] = q.mt;
    lds[w][4] = q.st;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int k = 1; k < kKlThreads / kWave; ++k) {
      KlState other{lds[k][0], lds[k][1], lds[k][2], lds[k][3], lds[k][4]};
      merge_kl(q, other);
    }
    const KlRow r = kl_finish(q);
    kl[tok] = r.kl;
    lse_s[tok] = r.lse_s;
    lse_t[tok] = r.lse_t;
  }
}

// The same backward as one-shot workgroups of 256 threads that each take 4 KB of a row (one 16-byte vector of both
// inputs per thread) in address order and exit: the form the memory system serves fastest when nothing has to stay on
// chip between a row's reads and its write.  Rows without gradient are written as zeros without a read.
constexpr int kKlChunkThreads = 256;
template <typename T>
__global__ __launch_bounds__(kKlChunkThreads) void reverse_kl_bwd_chunk_kernel(
    const T* __restrict__ student, const T* __restrict__ teacher, int64_t stride, int64_t nvec, unsigned chunks_per_row,
    const float* __restrict__ kl, const float* __restrict__ lse_s, const float* __restrict__ lse_t,
    const float* __restrict__ g, float grad_scale, const float* __restrict__ grad_scale_dev,
    T* __restrict__ dstudent) {
  constexpr int VN = Row<T>::kPerVec;
  const unsigned b = blockIdx.x;
  const unsigned tok = b / chunks_per_row, chunk = b - tok * chunks_per_row;
  const int64_t i = int64_t(chunk) * kKlChunkThreads + threadIdx.x;
  if (i >= nvec) return;
  u32x4* dv = reinterpret_cast<u32x4*>(dstudent + int64_t(tok) * stride);
  if (grad_scale_dev) grad_scale *= *grad_scale_dev;
  const float gt = g[tok] * grad_scale;
  if (gt == 0.f) {
    store_stream(dv + i, u32x4{0u, 0u, 0u, 0u});
    return;
  }
  const u32x4 rs = load_stream(reinterpret_cast<const u32x4*>(student + int64_t(tok) * stride) + i);
  const u32x4 rt = load_stream(reinterpret_cast<const u32x4*>(teacher + int64_t(tok) * stride) + i);
  const float k0 = -lse_s[tok] * kLog2e;
  const float k1 = gt * (lse_t[tok] - lse_s[tok] - kl[tok]);
  float a[VN], bb[VN];
  Row<T>::unpack(rs, a);
  Row<T>::unpack(rt, bb);
#pragma unroll
  for (int k = 0; k < VN; ++k) a[k] = fast_exp2(fmaf(a[k], kLog2e, k0)) * fmaf(a[k] - bb[k], gt, k1);
  store_stream(dv + i, Row<T>::pack(a));
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kKlThreads) void reverse_kl_bwd_kernel(
    const T* __restrict__ student, const T* __restrict__ teacher, int64_t stride, int64_t vocab,
    const float* __restrict__ kl, const float* __restrict__ lse_s, const float* __restrict__ lse_t,
    const float* __restrict__ g, float grad_scale, const float* __restrict__ grad_scale_dev,
    T* __restrict__ dstudent) {
  const int64_t tok = blockIdx.x;
  T* d = dstudent + tok * stride;
  if (grad_scale_dev) grad_scale *= *grad_scale_dev;
  const float gt = g[tok] * grad_scale;
  if (gt == 0.f) {
    if (VEC) {
      constexpr int VN = Row<T>::kPerVec;
      const int64_t nvec = vocab / VN;
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (int64_t i = threadIdx.x; i < nvec; i += kKlThreads) store_stream(reinterpret_cast<u32x4*>(d) + i, z);
      for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kKlThreads) Row<T>::store1(d + e, 0.f);
    } else {
      for (int64_t e = threadIdx.x; e < vocab; e += kKlThreads) Row<T>::store1(d + e, 0.f);
    }
    return;
  }
  const T* xs = student + tok * stride;
  const T* xt = teacher + tok * stride;
  const float k0 = -lse_s[tok] * kLog2e;
  const float k1 = gt * (lse_t[tok] - lse_s[tok] - kl[tok]);
  // d = p_s * g * ((x_s - x_t) + lse_t - lse_s - KL)
  if (VEC) {
    constexpr int VN = Row<T>::kPerVec;
    const u32x4* sv = reinterpret_cast<const u32x4*>(xs);
    const u32x4* tv = reinterpret_cast<const u32x4*>(xt);
    u32x4* dv = reinterpret_cast<u32x4*>(d);
    const int64_t nvec = vocab / VN;
    int64_t i = threadIdx.x;
    for (; i + int64_t(kKlUnroll - 1) * kKlThreads < nvec; i += int64_t(kKlUnroll) * kKlThreads) {
      u32x4 rs[kKlUnroll], rt[kKlUnroll];
#pragma unroll
      for (int u = 0; u < kKlUnroll; ++u) {
        rs[u] = load_stream(sv + i + int64_t(u) * kKlThreads);
        rt[u] = load_stream(tv + i + int64_t(u) * kKlThreads);
      }
#pragma unroll
      for (int u = 0; u < kKlUnroll; ++u) {
        float a[VN], b[VN];
        Row<T>::unpack(rs[u], a);
        Row<T>::unpack(rt[u], b);
#pragma unroll
        for (int k = 0; k < VN; ++k) a[k] = fast_exp2(fmaf(a[k], kLog2e, k0)) * fmaf(a[k] - b[k], gt, k1);
        store_stream(dv + i + int64_t(u) * kKlThreads, Row<T>::pack(a));
      }
    }
    for (; i < nvec; i += kKlThreads) {
      float a[VN], b[VN];
      Row<T>::unpack(load_stream(sv + i), a);
      Row<T>::unpack(load_stream(tv + i), b);
#pragma unroll
      for (int k = 0; k < VN; ++k) a[k] = fast_exp2(fmaf(a[k], kLog2e, k0)) * fmaf(a[k] - b[k], gt, k1);
      store_stream(dv + i, Row<T>::pack(a));
    }
    for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kKlThreads) {
      const float a = Row<T>::load1(xs + e), b = Row<T>::load1(xt + e);
      Row<T>::store1(d + e, fast_exp2(fmaf(a, kLog2e, k0)) * fmaf(a - b, gt, k1));
    }
  } else {
    for (int64_t e = threadIdx.x; e < vocab; e += kKlThreads) {
      const float a = Row<T>::load1(xs + e), b = Row<T>::load1(xt + e);
      Row<T>::store1(d + e, fast_exp2(fmaf(a, kLog2e, k0)) * fmaf(a - b, gt, k1));
    }
  }
}

// Forward + backward in ONE launch for a loss whose gradient w.r.t. each token's KL is known up front (masked token
// mean: g = mask / max(sum mask, 1)).  The workgroup scans the student and teacher rows with ordinary (cached) loads,
// thread 0 finishes KL / lse_s / lse_t, and the workgroup walks both rows again at once -- served by L2 / the
// memory-side cache -- to stream the student gradient out.  HBM sees 3*V*s bytes per token instead of 5*V*s.
// Tokens with g == 0 still report their KL but get a zero gradient row without a second walk.
template <typename T, bool VEC, int THREADS>
__global__ __launch_bounds__(THREADS) void reverse_kl_step_kernel(
    const T* __restrict__ student, const T* __restrict__ teacher, int64_t stride, int64_t vocab,
    const float* __restrict__ g, float grad_scale, float* __restrict__ kl, float* __restrict__ lse_s,
    float* __restrict__ lse_t, T* __restrict__ dstudent) {
  __shared__ float lds[THREADS / kWave][5];
  __shared__ float bc[2];
  const int tid = threadIdx.x;
  const int64_t tok = blockIdx.x;
  const T* xs = student + tok * stride;
  const T* xt = teacher + tok * stride;
  T* d = dstudent + tok * stride;
  const float gt = g[tok] * grad_scale;
  KlState q{kNegHuge, 0.f, 0.f, kNegHuge, 0.f};
  constexpr int VN = Row<T>::kPerVec;
  const int64_t nvec = VEC ? vocab / VN : 0;
  if (VEC) {
    const u32x4* sv = reinterpret_cast<const u32x4*>(xs);
    const u32x4* tv = reinterpret_cast<const u32x4*>(xt);
    int64_t i = tid;
    for (; i + int64_t(kKlUnroll - 1) * THREADS < nvec; i += int64_t(kKlUnroll) * THREADS) {
      u32x4 rs[kKlUnroll], rt[kKlUnroll];
#pragma unroll
      for (int u = 0; u < kKlUnroll; ++u) {
        rs[u] = sv[i + int64_t(u) * THREADS];
        rt[u] = tv[i + int64_t(u) * THREADS];
      }
      float a[kKlUnroll * VN], b[kKlUnroll * VN];
#pragma unroll
      for (int u = 0; u < kKlUnroll; ++u) {
        float pa[VN], pb[VN];
        Row<T>::unpack(rs[u], pa);
        Row<T>::unpack(rt[u], pb);
#pragma unroll
        for (int k = 0; k < VN; ++k) {
          a[u * VN + k] = pa[k];
          b[u * VN + k] = pb[k];
        }
      }
      absorb_pair(a, b, q);
    }
    for (; i < nvec; i += THREADS) {
      float a[VN], b[VN];
      Row<T>::unpack(sv[i], a);
      Row<T>::unpack(tv[i], b);
      absorb_pair(a, b, q);
    }
  }
  for (int64_t e = nvec * VN + tid; e < vocab; e += THREADS) {
    float a[1] = {Row<T>::load1(xs + e)}, b[1] = {Row<T>::load1(xt + e)};
    absorb_pair(a, b, q);
  }
  wave_butterfly([&](auto o) {
    constexpr int O = decltype(o)::value;
    KlState other{lane_xor<O>(q.ms), lane_xor<O>(q.ss), lane_xor<O>(q.us), lane_xor<O>(q.mt), lane_xor<O>(q.st)};
    merge_kl(q, other);
  });
  const int lane = tid & (kWave - 1), w = tid / kWave;
  if (lane == 0) {
    lds[w][0] = q.ms;
    lds[w][1] = q.ss;
    lds[w][2] = q.us;
    lds[w][3] = q.mt;
    lds[w][4] = q.st;
  }
  __syncthreads();
  if (tid == 0) {
    for (int k = 1; k < THREADS / kWave; ++k) {
      KlState other{lds[k][0], lds[k][1], lds[k][2], lds[k][3], lds[k][4]};
      merge_kl(q, other);
    }
    const KlRow r = kl_finish(q);
    const float ls = r.lse_s, lt = r.lse_t, v = r.kl;
    kl[tok] = v;
    lse_s[tok] = ls;
    lse_t[tok] = lt;
    bc[0] = -ls * kLog2e;
    bc[1] = gt * (lt - ls - v);
  }
  __syncthreads();
  const float k0 = bc[0], k1 = bc[1];
  // d = p_s * g * ((x_s - x_t) + lse_t - lse_s - KL); last use of both rows: non-temporal loads
  if (VEC) {
    const u32x4* sv = reinterpret_cast<const u32x4*>(xs);
    const u32x4* tv = reinterpret_cast<const u32x4*>(xt);
    u32x4* dv = reinterpret_cast<u32x4*>(d);
    if (gt == 0.f) {
      const u32x4 z = {0u, 0u, 0u, 0u};
      for (int64_t i = tid; i < nvec; i += THREADS) store_stream(dv + i, z);
    } else {
      // from the rows' end to their beginning: the second walk starts on what the caches still hold from the scan.
      // The lane's share is the scan's: `nfull` batches of kKlUnroll vectors at a stride of THREADS, then singles.
      const int64_t nfull = nvec > int64_t(kKlUnroll - 1) * THREADS + tid
                                ? (nvec - int64_t(kKlUnroll - 1) * THREADS - tid - 1) / (int64_t(kKlUnroll) * THREADS) + 1
                                : 0;
      const int64_t single0 = int64_t(tid) + nfull * kKlUnroll * THREADS;
      const int64_t nsingle = single0 < nvec ? (nvec - single0 - 1) / THREADS + 1 : 0;
      for (int64_t q2 = nsingle - 1; q2 >= 0; --q2) {
        const int64_t i = single0 + q2 * THREADS;
        float a[VN], b[VN];
        Row<T>::unpack(load_stream(sv + i), a);
        Row<T>::unpack(load_stream(tv + i), b);
#pragma unroll
        for (int k = 0; k < VN; ++k) a[k] = fast_exp2(fmaf(a[k], kLog2e, k0)) * fmaf(a[k] - b[k], gt, k1);
        store_stream(dv + i, Row<T>::pack(a));
      }
      for (int64_t bi = nfull - 1; bi >= 0; --bi) {
        const int64_t i = int64_t(tid) + bi * kKlUnroll * THREADS;
        u32x4 rs[kKlUnroll], rt[kKlUnroll];
#pragma unroll
        for (int u = kKlUnroll - 1; u >= 0; --u) {
          rs[u] = load_stream(sv + i + int64_t(u) * THREADS);
          rt[u] = load_stream(tv + i + int64_t(u) * THREADS);
        }
#pragma unroll
        for (int u = kKlUnroll - 1; u >= 0; --u) {
          float a[VN], b[VN];
          Row<T>::unpack(rs[u], a);
          Row<T>::unpack(rt[u], b);
#pragma unroll
          for (int k = 0; k < VN; ++k) a[k] = fast_exp2(fmaf(a[k], kLog2e, k0)) * fmaf(a[k] - b[k], gt, k1);
          store_stream(dv + i + int64_t(u) * THREADS, Row<T>::pack(a));
        }
      }
    }
  }
  for (int64_t e = nvec * VN + tid; e < vocab; e += THREADS) {
    const float a = Row<T>::load1(xs + e), b = Row<T>::load1(xt + e);
    Row<T>::store1(d + e, gt == 0.f ? 0.f : fast_exp2(fmaf(a, kLog2e, k0)) * fmaf(a - b, gt, k1));
  }
}

template <typename T>
static int launch_kl_step(const void* s, const void* t, int64_t n, int64_t vocab, int64_t stride, const float* g,
                          float scale, float* kl, float* ls, float* lt, void* d, hipStream_t st) {
  const bool vec = aligned16(s) && aligned16(t) && aligned16(d) && (stride * int64_t(sizeof(T))) % 16 == 0;
  dim3 grid(static_cast<unsigned>(n));
  // relax_amd_set_kernel_choice: TWO_WALK = the two-walk kernel for every row length; RESIDENT = fail where the
  // register-resident one is not built
  const int choice = kernel_choice();
  if (vec && choice == RELAX_AMD_KERNEL_AUTO) {  // one-shot workgroups that share each row
    const int rc = launch_reverse_kl_split<T>(static_cast<const T*>(s), static_cast<const T*>(t), stride, vocab, n, g,
                                              scale, kl, ls, lt, static_cast<T*>(d), st);
    if (rc != RELAX_AMD_EUNSUPPORTED) return rc;
  }
  if (vec && choice != RELAX_AMD_KERNEL_TWO_WALK) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    const int rc = launch_reverse_kl_resident<T>(static_cast<const T*>(s), static_cast<const T*>(t), stride, vocab, n,
                                                 g, scale, kl, ls, lt, static_cast<T*>(d), cus, st);
    if (rc != RELAX_AMD_EUNSUPPORTED) return rc;  // launched (or failed to): otherwise the row length is not built
  }
  if (choice == RELAX_AMD_KERNEL_RESIDENT) {  // a comparison of the two kernels must not pass on one of them
    set_error("reverse_kl_step_fused: kernel choice RESIDENT, but no register-resident kernel is built "
              "for rows of %lld elements of this type and alignment", (long long)vocab);
    return RELAX_AMD_EUNSUPPORTED;
  }
#define RELAX_AMD_KL_STEP(V, TH)                                                                                   \
  hipLaunchKernelGGL((reverse_kl_step_kernel<T, V, TH>), grid, dim3(TH), 0, st, static_cast<const T*>(s),            \
                     static_cast<const T*>(t), stride, vocab, g, scale, kl, ls, lt, static_cast<T*>(d))
  if (!vec) {
    RELAX_AMD_KL_STEP(false, 256);
  } else if (vocab / Row<T>::kPerVec >= 2048) {  // enough 16-byte vectors to keep 1024 threads busy
    RELAX_AMD_KL_STEP(true, 1024);
  } else {
    RELAX_AMD_KL_STEP(true, 256);
  }
#undef RELAX_AMD_KL_STEP
  return check_launch("reverse_kl_step_fused");
}

template <typename T>
static int launch_kl_fwd(const void* s, const void* t, int64_t n, int64_t vocab, int64_t stride, float* kl,
                         float* ls, float* lt, hipStream_t st) {
  const bool vec = aligned16(s) && aligned16(t) && (stride * int64_t(sizeof(T))) % 16 == 0;
  dim3 grid(static_cast<unsigned>(n)), block(kKlThreads);
  if (vec)
    hipLaunchKernelGGL((reverse_kl_fwd_kernel<T, true>), grid, block, 0, st, static_cast<const T*>(s),
                       static_cast<const T*>(t), stride, vocab, kl, ls, lt);
  else
    hipLaunchKernelGGL((reverse_kl_fwd_kernel<T, false>), grid, block, 0, st, static_cast<const T*>(s),
                       static_cast<const T*>(t), stride, vocab, kl, ls, lt);
  return check_launch("reverse_kl_fwd");
}

template <typename T>
static int launch_kl_bwd(const void* s, const void* t, int64_t n, int64_t vocab, int64_t stride, const float* kl,
                         const float* ls, const float* lt, const float* g, float scale, const float* scale_dev,
                         void* d, hipStream_t st) {
  const bool vec = aligned16(s) && aligned16(t) && aligned16(d) && (stride * int64_t(sizeof(T))) % 16 == 0;
  dim3 grid(static_cast<unsigned>(n)), block(kKlThreads);
  // rows of whole 16-byte vectors: the chunk form (same bits); relax_amd_set_kernel_choice(TWO_WALK) keeps the
  // row-per-workgroup loop for comparisons
  if (vec && vocab % Row<T>::kPerVec == 0 && kernel_choice() != RELAX_AMD_KERNEL_TWO_WALK) {
    const int64_t nvec = vocab / Row<T>::kPerVec;
    const int64_t chunks = (nvec + kKlChunkThreads - 1) / kKlChunkThreads;
    if (n * chunks <= 2147483647LL) {
      hipLaunchKernelGGL((reverse_kl_bwd_chunk_kernel<T>), dim3(static_cast<unsigned>(n * chunks)),
                         dim3(kKlChunkThreads), 0, st, static_cast<const T*>(s), static_cast<const T*>(t), stride, nvec,
                         static_cast<unsigned>(chunks), kl, ls, lt, g, scale, scale_dev, static_cast<T*>(d));
      return check_launch("reverse_kl_bwd_chunk");
    }
  }
  if (vec)
    hipLaunchKernelGGL((reverse_kl_bwd_kernel<T, true>), grid, block, 0, st, static_cast<const T*>(s),
                       static_cast<const T*>(t), stride, vocab, kl, ls, lt, g, scale, scale_dev, static_cast<T*>(d));
  else
    hipLaunchKernelGGL((reverse_kl_bwd_kernel<T, false>), grid, block, 0, st, static_cast<const T*>(s),
                       static_cast<const T*>(t), stride, vocab, kl, ls, lt, g, scale, scale_dev, static_cast<T*>(d));
  return check_launch("reverse_kl_bwd");
}

}  // namespace relax_amd

using namespace relax_amd;

static int kl_check(const char* what, int64_t n, int64_t vocab, int64_t stride) {
  if (n < 0 || n > 2147483647LL || vocab <= 0 || stride < vocab) {
    set_error("%s: bad shape n_tokens=%lld vocab=%lld row_stride=%lld", what, (long long)n, (long long)vocab,
              (long long)stride);
    return RELAX_AMD_EINVAL;
  }
  return RELAX_AMD_OK;
}

extern "C" int relax_amd_reverse_kl_fwd(const void* student, const void* teacher, int dtype, int64_t n_tokens,
                                        int64_t vocab, int64_t row_stride, float* kl, float* lse_s, float* lse_t,
                                        void* stream) {
  if (int rc = kl_check("reverse_kl_fwd", n_tokens, vocab, row_stride)) return rc;
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (!student || !teacher || !kl || !lse_s || !lse_t) {
    set_error("reverse_kl_fwd: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32: return launch_kl_fwd<float>(student, teacher, n_tokens, vocab, row_stride, kl, lse_s, lse_t, s);
    case RELAX_AMD_BF16: return launch_kl_fwd<bf16_t>(student, teacher, n_tokens, vocab, row_stride, kl, lse_s, lse_t,
        s);
    case RELAX_AMD_F16: return launch_kl_fwd<f16_t>(student, teacher, n_tokens, vocab, row_stride, kl, lse_s, lse_t, s);
    default: set_error("reverse_kl_fwd: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
}

extern "C" int relax_amd_reverse_kl_bwd(const void* student, const void* teacher, int dtype, int64_t n_tokens,
                                        int64_t vocab, int64_t row_stride, const float* kl, const float* lse_s,
                                        const float* lse_t, const float* g, float grad_scale,
                                        const float* grad_scale_dev, void* dstudent, void* stream) {
  if (int rc = kl_check("reverse_kl_bwd", n_tokens, vocab, row_stride)) return rc;
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (!student || !teacher || !kl || !lse_s || !lse_t || !g || !dstudent) {
    set_error("reverse_kl_bwd: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32:
      return launch_kl_bwd<float>(student, teacher, n_tokens, vocab, row_stride, kl, lse_s, lse_t, g, grad_scale,
          grad_scale_dev, dstudent, s);
    case RELAX_AMD_BF16:
      return launch_kl_bwd<bf16_t>(student, teacher, n_tokens, vocab, row_stride, kl, lse_s, lse_t, g, grad_scale,
          grad_scale_dev, dstudent, s);
    case RELAX_AMD_F16:
      return launch_kl_bwd<f16_t>(student, teacher, n_tokens, vocab, row_stride, kl, lse_s, lse_t, g, grad_scale,
          grad_scale_dev, dstudent, s);
    default: set_error("reverse_kl_bwd: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
}

extern "C" int relax_amd_reverse_kl_step_fused(const void* student, const void* teacher, int dtype, int64_t n_tokens,
                                               int64_t vocab, int64_t row_stride, const float* g, float grad_scale,
                                               float* kl, float* lse_s, float* lse_t, void* dstudent, void* stream) {
  if (int rc = kl_check("reverse_kl_step_fused", n_tokens, vocab, row_stride)) return rc;
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (!student || !teacher || !g || !kl || !lse_s || !lse_t || !dstudent) {
    set_error("reverse_kl_step_fused: NULL argument");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32:
      return launch_kl_step<float>(student, teacher, n_tokens, vocab, row_stride, g, grad_scale, kl, lse_s, lse_t,
          dstudent, s);
    case RELAX_AMD_BF16:
      return launch_kl_step<bf16_t>(student, teacher, n_tokens, vocab, row_stride, g, grad_scale, kl, lse_s, lse_t,
          dstudent, s);
    case RELAX_AMD_F16:
      return launch_kl_step<f16_t>(student, teacher, n_tokens, vocab, row_stride, g, grad_scale, kl, lse_s, lse_t,
          dstudent, s);
    default: set_error("reverse_kl_step_fused: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
}
