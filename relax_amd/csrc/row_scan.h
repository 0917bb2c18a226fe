// Online-softmax row scan shared by the forward-only log-prob kernel and the fused actor-step kernel.  Both kernels
// take the same path through this file with the same workgroup shape for a given row length, so for one logits row
// they produce bit-identical (max, sum exp, sum exp*x): the forward-only pass (old / reference log-probs) and the
// training forward then agree exactly, which Relax's step-0 check (ppo_kl == 0 for identical weights) relies on.
// Wherever a product feeds a sum the fused multiply-add is written out, so that no context-dependent contraction of a
// separate multiply and add can creep in.
#pragma once

#include "device_utils.h"

namespace relax_amd {

constexpr int kScanUnroll = 4;  // 16-byte loads in flight per lane

struct SoftmaxAcc {
  float m, s, t;  // max of x*c, sum exp2(x*c - m), sum exp2(x*c - m) * x     (c = log2(e) / temperature)
};

// Returns the largest of the K values (a float maximum: NaN passes unnoticed here and shows in st.s instead).
// WITH_T = false leaves st.t alone (callers that want neither the entropy nor sum p*x: one multiply-add per element
// less); st.m and st.s, and with them the log-sum-exp, are the same bits either way.
template <int K, bool WITH_T = true>
__device__ __forceinline__ float scan_absorb(const float (&v)[K], float c, SoftmaxAcc& st) {
  float vmax = v[0];
#pragma unroll
  for (int i = 1; i < K; ++i) vmax = fmaxf(vmax, v[i]);
  const float mc = __fmul_rn(vmax, c);
  if (mc > st.m) {
    const float sc = fast_exp2(fmaf(-vmax, c, st.m));  // one rounding, spelled out (see scan_finish)
    st.s = __fmul_rn(st.s, sc);
    if (WITH_T) st.t = __fmul_rn(st.t, sc);
    st.m = mc;
  }
#pragma unroll
  for (int i = 0; i < K; ++i) {
    const float e = fast_exp2(fmaf(v[i], c, -st.m));
    st.s = __fadd_rn(st.s, e);
    if (WITH_T) st.t = fmaf(e, v[i], st.t);
  }
  return vmax;
}

__device__ __forceinline__ void scan_merge(SoftmaxAcc& a, float m2, float s2, float t2) {
  const float mn = fmaxf(a.m, m2);
  const float fa = fast_exp2(__fsub_rn(a.m, mn)), fb = fast_exp2(__fsub_rn(m2, mn));
  a.s = fmaf(a.s, fa, __fmul_rn(s2, fb));
  a.t = fmaf(a.t, fa, __fmul_rn(t2, fb));
  a.m = mn;
}

// Optional observer of the scan: is told the largest value of every batch of elements a lane absorbs (kScanUnroll
// vectors at a stride of THREADS vectors while that many remain, then single vectors, then single tail elements), in
// the order scan_row() takes them, without touching the softmax arithmetic or its order.
struct ScanNoHook {
  __device__ __forceinline__ void absorbed(float) const {}
};

// Per-lane state over one row.  VEC: 16-byte loads (row base and stride 16-byte aligned) for the whole vectors and
// scalar loads for the tail; otherwise scalar loads throughout.  STREAM selects non-temporal loads (row not needed
// again soon) or ordinary cached loads (a second pass over the row follows immediately); it does not change results.
template <typename T, bool VEC, bool STREAM, int THREADS, typename Hook = ScanNoHook, bool WITH_T = true>
__device__ __forceinline__ SoftmaxAcc scan_row(const T* __restrict__ x, int64_t vocab, float c, Hook&& hook = Hook()) {
  SoftmaxAcc st{kNegHuge, 0.f, 0.f};
  if (VEC) {
    constexpr int VN = Row<T>::kPerVec;
    const u32x4* xv = reinterpret_cast<const u32x4*>(x);
    const int64_t nvec = vocab / VN;
    int64_t i = threadIdx.x;
    for (; i + int64_t(kScanUnroll - 1) * THREADS < nvec; i += int64_t(kScanUnroll) * THREADS) {
      u32x4 raw[kScanUnroll];
#pragma unroll
      for (int u = 0; u < kScanUnroll; ++u)
        raw[u] = STREAM ? load_stream(xv + i + int64_t(u) * THREADS) : xv[i + int64_t(u) * THREADS];
      float v[kScanUnroll * VN];
#pragma unroll
      for (int u = 0; u < kScanUnroll; ++u) {
        float part[VN];
        Row<T>::unpack(raw[u], part);
#pragma unroll
        for (int k = 0; k < VN; ++k) v[u * VN + k] = part[k];
      }
      hook.absorbed(scan_absorb<sizeof(v) / sizeof(float), WITH_T>(v, c, st));
    }
    for (; i < nvec; i += THREADS) {
      float v[VN];
      Row<T>::unpack(STREAM ? load_stream(xv + i) : xv[i], v);
      hook.absorbed(scan_absorb<sizeof(v) / sizeof(float), WITH_T>(v, c, st));
    }
    for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += THREADS) {
      float v[1] = {Row<T>::load1(x + e)};
      hook.absorbed(scan_absorb<sizeof(v) / sizeof(float), WITH_T>(v, c, st));
    }
  } else {
    for (int64_t e = threadIdx.x; e < vocab; e += THREADS) {
      float v[1] = {Row<T>::load1(x + e)};
      hook.absorbed(scan_absorb<sizeof(v) / sizeof(float), WITH_T>(v, c, st));
    }
  }
  return st;
}

// Wave64 xor-butterfly, then waves in index order through LDS; the merged state is valid in thread 0 only.
template <int THREADS>
__device__ __forceinline__ void scan_block_merge(SoftmaxAcc& st, float (*wave_state)[3]) {
  wave_butterfly([&](auto o) {
    constexpr int O = decltype(o)::value;
    scan_merge(st, lane_xor<O>(st.m), lane_xor<O>(st.s), lane_xor<O>(st.t));
  });
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  if (lane == 0) {
    wave_state[wave][0] = st.m;
    wave_state[wave][1] = st.s;
    wave_state[wave][2] = st.t;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
#pragma unroll
    for (int i = 1; i < THREADS / kWave; ++i) scan_merge(st, wave_state[i][0], wave_state[i][1], wave_state[i][2]);
  }
}

// lse = logsumexp(x/T), spx = sum_v softmax * (x/T), entropy = lse - spx, lp = x_target/T - lse
__device__ __forceinline__ void scan_finish(const SoftmaxAcc& st, float x_target, bool target_ok, float inv_t,
                                            float& lse, float& spx, float& ent, float& lp) {
  lse = fmaf(st.m, kLn2, logf(st.s));
  const float q = __fdiv_rn(st.t, st.s);
  spx = __fmul_rn(q, inv_t);
  // A product feeding a sum is written as the fused multiply-add it may become: __fmul_rn / __fsub_rn are a plain
  // `*` / `-` to this compiler, which contracts them or not depending on the code around the call, so lse - q * inv_t
  // came out with one rounding in some kernels and two in others when the temperature is not 1.
  ent = fmaf(-q, inv_t, lse);
  lp = target_ok ? fmaf(x_target, inv_t, -lse) : __builtin_nanf("");
}

// Workgroup width for a row of `vocab` elements: wide workgroups for long rows (fewer rows in flight, so the second
// pass of the fused kernel finds its row still cached), narrow ones for short rows.  One rule for every kernel.
// (1024 from seven vectors per thread on: fp32 rows of 32000 entries, 8000 vectors, then fit one 1024-thread
// workgroup per CU of the register-resident kernels, which streams 4 % faster than two 512-thread ones.)
inline int scan_threads(int64_t vocab, int per_vec) {
  const int64_t nvec = vocab / per_vec;
  if (nvec >= 7168) return 1024;
  if (nvec >= 2048) return 512;
  return 256;
}

}  // namespace relax_amd
