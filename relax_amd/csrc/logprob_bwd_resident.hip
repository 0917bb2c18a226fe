// dlogits backward of the log-prob / entropy pair in the burst form of the register-resident actor step: persistent
// workgroups (one of 1024 threads per CU), each taking a whole row into its
// registers in one burst of loads, turning it into its gradient in place and writing it out in one burst of stores.
// Same arithmetic, element by element, as logprob_entropy_bwd_kernel (logprob_entropy.hip):
//   d = inv_t * p * (-g_lp + g_H * (spx - x * inv_t))  (+ inv_t * g_lp at the target),  p = exp(x * inv_t - lse),
// so both return the same bits; rows without gradient are zero-filled without being read.  What differs is the
// order of the memory requests: the row-per-workgroup grid interleaves four loads with four stores from thousands of
// workgroups, this one sends 304 KB of one kind at a time from each CU, which is what the memory system serves
// fastest (see actor_step_resident.hip).
//
// Replaces, like logprob_entropy_bwd_kernel, _VocabParallelLogProbEntropy.backward
// (relax/utils/training/ppo_utils.py:560-629) for one micro-batch.
//
// hipcc-flags: -mllvm -amdgpu-use-amdgpu-trackers=1
#include "logprob_bwd_resident.h"

#include "device_utils.h"
#include "row_scan.h"

namespace relax_amd {

// Workgroup width, as in the register-resident actor step.
template <typename T>
constexpr int bwd_resident_threads() {
  return 1024;
}

template <typename T, int NVF, bool PARTIAL>
__global__ __launch_bounds__(bwd_resident_threads<T>(), 4) void logprob_entropy_bwd_resident_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
    const int32_t* __restrict__ token_of_row, const int64_t* __restrict__ targets, const float* __restrict__ lse,
    const float* __restrict__ spx, const float* __restrict__ g_lp, const float* __restrict__ g_ent, float grad_scale,
    const float* __restrict__ grad_scale_dev, float c, float inv_t, T* __restrict__ dlogits, int64_t d_stride) {
  constexpr int THREADS = bwd_resident_threads<T>();
  constexpr int VN = Row<T>::kPerVec;
  constexpr int NV = NVF + (PARTIAL ? 1 : 0);  // vector positions per thread
  __shared__ float bc[4];
  __shared__ int64_t bc_target;
  const int tid = threadIdx.x;
  const int rem = int(vocab / VN) - NVF * THREADS;  // lanes that hold a vector at the partial position (host-checked)
  if (grad_scale_dev) grad_scale *= *grad_scale_dev;
  u32x4 reg[NV];

  // does this lane hold a vector at position j?  A compile-time answer except at the partial position.
  auto has = [&](int j) -> bool { return j < NVF || (PARTIAL && j == NVF && tid < rem); };
  // token of a row, or -1 when the row has no gradient (it scores nothing, or both coefficients vanish); uniform over
  // the workgroup
  auto live_token = [&](int64_t row) -> int64_t {
    if (row >= n_rows) return -1;
    const int64_t tok = token_of_row ? int64_t(token_of_row[row]) : row;
    if (tok < 0) return -1;
    const float glp = g_lp[tok] * grad_scale;
    const float gh = g_ent ? g_ent[tok] * grad_scale : 0.f;
    return (glp == 0.f && gh == 0.f) ? -1 : tok;
  };
  auto zero_fill = [&](int64_t row) {
    u32x4* dv = reinterpret_cast<u32x4*>(dlogits + row * d_stride);
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (has(j)) store_stream(dv + tid + j * THREADS, u32x4{0u, 0u, 0u, 0u});
  };
  // this workgroup's first row with a gradient at or after `row` (n_rows or more: none); the rows passed on the way
  // are zero-filled here
  auto advance = [&](int64_t row) -> int64_t {
    while (row < n_rows && live_token(row) < 0) {
      zero_fill(row);
      row += gridDim.x;
    }
    return row;
  };

  int64_t row = advance(blockIdx.x);
  if (row >= n_rows) return;
  int64_t tok = live_token(row);
  {
    const u32x4* xv = reinterpret_cast<const u32x4*>(logits + row * row_stride);
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (has(j)) reg[j] = load_stream(xv + tid + j * THREADS);
  }
  while (true) {
    const int64_t next = advance(row + gridDim.x);
    const bool has_next = next < n_rows;
    const int64_t next_tok = has_next ? live_token(next) : -1;
    // the row's constants, as logprob_entropy_bwd_kernel forms them, by thread 0 and through LDS to everyone: the
    // barrier also keeps the waves of the workgroup in step, so that its stores and loads go out as one burst each
    // (and its fence waits for this wave's loads: the row is complete in the registers behind it)
    if (tid == 0) {
      const float glp = g_lp[tok] * grad_scale;
      const float gh = g_ent ? g_ent[tok] * grad_scale : 0.f;
      const float b = gh * inv_t;
      bc[0] = -lse[tok] * kLog2e;                                    // k0: p = exp2(x*c + k0)
      bc[1] = -glp * inv_t + (gh != 0.f ? b * spx[tok] : 0.f);       // a0
      bc[2] = -b * inv_t;                                            // a1: d = p * (a0 + a1*x)
      bc[3] = glp * inv_t;                                           // added at the target
      bc_target = targets[tok];
    }
    __syncthreads();
    const float k0 = bc[0], a0 = bc[1], a1 = bc[2], hot = bc[3];
    const int64_t tg = bc_target;
    const int tvec = (tg >= 0 && tg < vocab) ? int(tg / VN) : -1;
    const int tsub = int(tg % VN);
    __syncthreads();  // everyone has read the constants before thread 0 writes the next row's
    // the row becomes its gradient in place ...
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));  // recomputed per vector: loop-invariant index registers would not fit
      const int idx = lane_id + j * THREADS;
      // an opaque copy: unpacked next to the loads (where the compiler would otherwise move it, carrying eight floats
      // per vector around the loop instead of four words) the row no longer fits the registers
      asm volatile("" : "+v"(reg[j].x), "+v"(reg[j].y), "+v"(reg[j].z), "+v"(reg[j].w));
      float v[VN];
      Row<T>::unpack(reg[j], v);
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        v[k] = fast_exp2(fmaf(v[k], c, k0)) * fmaf(v[k], a1, a0);
        if (k == VN / 2 - 1) __builtin_amdgcn_sched_barrier(0);  // half a vector's temporaries at a time
      }
      // the target's element, in one lane of the workgroup per row: as selects (a branch around the update keeps the
      // eight values as one wide register tuple through the join, and the row no longer fits the registers)
      const int sub_here = idx == tvec ? tsub : -1;
#pragma unroll
      for (int k = 0; k < VN; ++k) v[k] = k == sub_here ? v[k] + hot : v[k];
      reg[j] = Row<T>::pack(v);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ... leaves in one burst of stores, and the next row with a gradient arrives in one burst of loads (without one
    // the row itself is read again: a branch here would cost the precise wait counts)
    u32x4* dv = reinterpret_cast<u32x4*>(dlogits + row * d_stride);
    const u32x4* nxv = reinterpret_cast<const u32x4*>(logits + (has_next ? next : row) * row_stride);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));
      if (has(j)) store_stream(dv + lane_id + j * THREADS, reg[j]);
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));
      if (has(j)) reg[j] = load_stream(nxv + lane_id + j * THREADS);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!has_next) return;
    row = next;
    tok = next_tok;
  }
}

#define RELAX_AMD_BWD_RESIDENT(NVF, PARTIAL)                                                                         \
  if (full == NVF && partial == PARTIAL) {                                                                            \
    hipLaunchKernelGGL((logprob_entropy_bwd_resident_kernel<T, NVF, PARTIAL>), grid, block, 0, stream, logits,       \
                       row_stride, vocab, n_rows, token_of_row, targets, lse, spx, g_lp, g_ent, grad_scale,          \
                       grad_scale_dev, inv_t * kLog2e, inv_t, dlogits, d_stride);                                    \
    return check_launch("logprob_entropy_bwd_resident");                                                             \
  }

template <typename T>
int launch_logprob_bwd_resident(const T* logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
                                const int32_t* token_of_row, const int64_t* targets, const float* lse,
                                const float* spx, const float* g_lp, const float* g_ent, float grad_scale,
                                const float* grad_scale_dev, float inv_t, T* dlogits, int64_t d_stride,
                                int compute_units, hipStream_t stream) {
  constexpr int VN = Row<T>::kPerVec, THREADS = bwd_resident_threads<T>();
  if (vocab % VN != 0) return RELAX_AMD_EUNSUPPORTED;
  const int64_t nvec = vocab / VN;
  const int full = int(nvec / THREADS);
  const bool partial = nvec % THREADS != 0;
  const int64_t slots = int64_t(compute_units) * (1024 / THREADS);  // persistent workgroups: as many as fit the chip
  const dim3 grid(static_cast<unsigned>(n_rows < slots ? n_rows : slots)), block(THREADS);
  if constexpr (sizeof(T) == 2) {
    // vocabularies of 163840 and up to it, 151936 / 152064, 128256 / 129280, 131072, 100352 / 102400 entries
    RELAX_AMD_BWD_RESIDENT(20, false)
    RELAX_AMD_BWD_RESIDENT(19, true)
    RELAX_AMD_BWD_RESIDENT(18, true)
    RELAX_AMD_BWD_RESIDENT(15, true)
    RELAX_AMD_BWD_RESIDENT(16, false)
    RELAX_AMD_BWD_RESIDENT(12, true)
    // 65536 and 57352 .. 65528 (64000)
    RELAX_AMD_BWD_RESIDENT(8, false)
    RELAX_AMD_BWD_RESIDENT(7, true)
  } else {
    // fp32 rows of 32000 entries, of 32768, of 49156 .. 53248, of 61444 .. 65532 and of 65536
    RELAX_AMD_BWD_RESIDENT(7, true)
    RELAX_AMD_BWD_RESIDENT(8, false)
    RELAX_AMD_BWD_RESIDENT(12, true)
    RELAX_AMD_BWD_RESIDENT(15, true)
    RELAX_AMD_BWD_RESIDENT(16, false)
  }
  return RELAX_AMD_EUNSUPPORTED;
}
#undef RELAX_AMD_BWD_RESIDENT

template int launch_logprob_bwd_resident<float>(const float*, int64_t, int64_t, int64_t, const int32_t*,
                                                const int64_t*, const float*, const float*, const float*,
                                                const float*, float, const float*, float, float*, int64_t, int,
                                                hipStream_t);
template int launch_logprob_bwd_resident<bf16_t>(const bf16_t*, int64_t, int64_t, int64_t, const int32_t*,
                                                 const int64_t*, const float*, const float*, const float*,
                                                 const float*, float, const float*, float, bf16_t*, int64_t, int,
                                                 hipStream_t);
template int launch_logprob_bwd_resident<f16_t>(const f16_t*, int64_t, int64_t, int64_t, const int32_t*,
                                                const int64_t*, const float*, const float*, const float*,
                                                const float*, float, const float*, float, f16_t*, int64_t, int,
                                                hipStream_t);

}  // namespace relax_amd
