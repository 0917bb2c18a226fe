// Register-resident fused reverse-KL step: the same computation as reverse_kl_step_kernel (per-token
// KL(student || teacher), both log-sum-exps and the student gradient for a known d loss / d KL, one launch) for long
// 16-bit rows of the common vocabulary sizes.
//
// A 1024-thread workgroup keeps the STUDENT row in its vector registers (19 16-byte vectors per thread at
// V = 151936) and streams the teacher row past it twice: once for the two online softmaxes, once for the gradient
// d = p_s * g * ((x_s - x_t) + lse_t - lse_s - KL).  HBM sees the student row once instead of twice (the two-walk
// kernel re-fetches ~85 % of both rows through the fabric).  Workgroups are persistent, one per CU, rows b, b + grid,
// ...; a row's gradient replaces the student row in the registers, leaves in one burst of stores, and the workgroup's
// next student row arrives in one burst of loads (with a store and a load alternating vector by vector behind the
// gradient arithmetic the launch took 2.97 ms on 16384 x 151936 rows instead of 2.84 ms: memory rewards the long
// bursts).  No workgroup waits for another; the loop bound is the only exit condition.
//
// As in the register-resident actor step, the row shape (NVF full vector positions per thread, plus a partially
// filled one when PARTIAL) is a template parameter so that every loop is straight-line code and the compiler can count
// how many loads and stores may stay in flight at each use, and the scan repeats the two-walk kernel's grouping and
// order (two vectors absorbed together while a thread has two to go, then single vectors; waves merged in index
// order), so both kernels return the same bits.
//
// Replaces, like the two-walk kernel, the jsd_alpha == 0 branch of compute_opd_kl on complete log-softmax rows
// (relax/utils/opd/opd_utils.py:1165-1169) and its autograd backward, for one micro-batch.
//
// hipcc-flags: -mllvm -amdgpu-use-amdgpu-trackers=1
#include "reverse_kl_resident.h"

#include <type_traits>

#include "device_utils.h"
#include "reverse_kl_math.h"

namespace relax_amd {

constexpr int kKlResThreads = 1024;
// Teacher vectors in flight ahead of their use.  The slots freed by a pass's last positions take the next pass's first
// vectors in rotated order, starting with vector NV % depth; the depth is chosen so that vector 0, needed first, is not
// the one requested last (which would make the next pass wait for everything in flight).
constexpr int kl_ring_depth(int nv) { return nv % 4 == 1 ? 5 : 4; }

// absorb_pair() over the values of kKlUnroll raw vector pairs, without holding them all unpacked
// marks a raw vector as changed without touching it: what is unpacked from it afterwards is a new value to the
// compiler, which would otherwise keep (and spill) the values unpacked earlier for the later uses
__device__ __forceinline__ void launder(u32x4& r) { asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w)); }

// vector `index` of the row at `row_base`: a wave-uniform base and a 32-bit per-lane byte offset, the addressing form
// that costs one vector register per access instead of a 64-bit per-lane pointer
template <typename P>
__device__ __forceinline__ P* row_vec(P* row_base, uint32_t index) {
  typedef typename std::conditional<std::is_const<P>::value, const char, char>::type Byte;
  return reinterpret_cast<P*>(reinterpret_cast<Byte*>(row_base) + index * uint32_t(sizeof(u32x4)));
}

template <typename T>
__device__ __forceinline__ void absorb_raw_pairs(u32x4* s_raw, u32x4** t_raw, KlState& q) {
  constexpr int VN = Row<T>::kPerVec;
  float smax = 0.f, tmax = 0.f;
#pragma unroll
  for (int u = 0; u < kKlUnroll; ++u) {
    float a[VN], b[VN];
    Row<T>::unpack(s_raw[u], a);
    Row<T>::unpack(*t_raw[u], b);
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      smax = (u == 0 && k == 0) ? a[0] : fmaxf(smax, a[k]);
      tmax = (u == 0 && k == 0) ? b[0] : fmaxf(tmax, b[k]);
    }
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
  for (int u = 0; u < kKlUnroll; ++u) {
    // unpack again: the values of the first walk kept alive (what common-subexpression elimination would do) do not
    // fit the register file next to the resident row
    launder(s_raw[u]);
    launder(*t_raw[u]);
    // one 32-bit word of the vectors at a time, in element order
    const uint32_t sw[4] = {s_raw[u].x, s_raw[u].y, s_raw[u].z, s_raw[u].w};
    const uint32_t tw[4] = {t_raw[u]->x, t_raw[u]->y, t_raw[u]->z, t_raw[u]->w};
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      float a[VN], b[VN];
      Row<T>::unpack(u32x4{sw[h], 0u, 0u, 0u}, a);
      Row<T>::unpack(u32x4{tw[h], 0u, 0u, 0u}, b);
#pragma unroll
      for (int k = 0; k < VN / 4; ++k) {
        const float es = fast_exp2(fmaf(a[k], kLog2e, -q.ms));
        const float et = fast_exp2(fmaf(b[k], kLog2e, -q.mt));
        q.ss += es;
        q.us = fmaf(es, a[k] - b[k], q.us);
        q.st += et;
      }
      if (h == 1) __builtin_amdgcn_sched_barrier(0);
    }
  }
}

template <typename T, int NVF, bool PARTIAL>
__global__ __launch_bounds__(kKlResThreads, 4) void reverse_kl_resident_kernel(
    const T* __restrict__ student, const T* __restrict__ teacher, int64_t stride, int64_t vocab, int64_t n_rows,
    const float* __restrict__ g, float grad_scale, float* __restrict__ kl, float* __restrict__ lse_s,
    float* __restrict__ lse_t, T* __restrict__ dstudent) {
  constexpr int THREADS = kKlResThreads, kU = kKlUnroll;
  constexpr int VN = Row<T>::kPerVec;
  constexpr int NV = NVF + (PARTIAL ? 1 : 0);  // vector positions per thread
  constexpr int D = kl_ring_depth(NV);
  constexpr int kGroups = (NV + kU - 1) / kU;
  static_assert(kU == 2 && D >= kU && D <= NVF, "the teacher ring is refilled pair by pair");
  __shared__ float lds[THREADS / kWave][5];
  __shared__ float bc[2];
  const int tid = threadIdx.x;
  const int rem = int(vocab / VN) - NVF * THREADS;  // lanes that hold a vector at the partial position (host-checked)
  u32x4 srow[NV];  // the student row
  u32x4 ring[D];   // teacher vectors in flight

  // does this lane hold a vector at position j?  A compile-time answer except at the partial position.
  auto has = [&](int j) -> bool { return j < NVF || (PARTIAL && j == NVF && tid < rem); };

  int64_t row = blockIdx.x;
  if (row >= n_rows) return;
  {
    const u32x4* sv = reinterpret_cast<const u32x4*>(student + row * stride);
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (has(j)) srow[j] = load_stream(row_vec(sv, tid + j * THREADS));
    const u32x4* tv0 = reinterpret_cast<const u32x4*>(teacher + row * stride);
#pragma unroll
    for (int j = 0; j < D; ++j) ring[j] = *row_vec(tv0, tid + j * THREADS);
  }

  while (true) {
    const int64_t next = row + gridDim.x;
    const bool has_next = next < n_rows;
    const float gt = g[row] * grad_scale;
    const u32x4* tv = reinterpret_cast<const u32x4*>(teacher + row * stride);

    // a token without gradient (g == 0) gets a zero row; the second pass's teacher loads then all go to the row's
    // first vector, which costs nothing, so that the instruction stream -- and with it the wait counts -- stays the same
    const bool emit_zero = gt == 0.f;
    const int tscale = emit_zero ? 0 : 1;

    // ---- scan: both online softmaxes and sum e_s * (x_s - x_t).  The teacher row streams through the ring (ordinary
    // loads: it is read again in a moment); its first D vectors are already on their way (requested during the previous
    // row's gradient pass), and the slots freed by the last D positions take the first vectors of the second pass, which
    // land during the merge.
    KlState q{kNegHuge, 0.f, 0.f, kNegHuge, 0.f};
    bool grouped = true;
#pragma unroll
    for (int gi = 0; gi < kGroups; ++gi) {
      const int j0 = kU * gi, j1 = kU * gi + 1;
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));  // recomputed per group: loop-invariant index registers would not fit
      if (grouped && j1 < NV && has(j1)) {
        u32x4* tpair[kU] = {&ring[j0 % D], &ring[j1 % D]};
        absorb_raw_pairs<T>(&srow[j0 < NV - 1 ? j0 : 0], tpair, q);
      } else {
        grouped = false;
#pragma unroll
        for (int u = 0; u < kU; ++u)
          if (j0 + u < NV && has(j0 + u)) {
            float a[VN], b[VN];
            launder(srow[j0 + u < NV ? j0 + u : NV - 1]);
            Row<T>::unpack(srow[j0 + u < NV ? j0 + u : NV - 1], a);
            Row<T>::unpack(ring[(j0 + u) % D], b);
            absorb_pair(a, b, q);
          }
      }
      // the ring slots just consumed take the vectors D positions further on, or the second pass's first ones
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int j = j0 + u;
        if (j >= NV) continue;
        if (j + D < NV) {
          if (has(j + D)) ring[j % D] = *row_vec(tv, lane_id + (j + D) * THREADS);
        } else {
          ring[j % D] = load_stream(row_vec(tv, (lane_id + (j % D) * THREADS) * tscale));
        }
      }
      asm volatile("" : "+v"(q.ss), "+v"(q.us), "+v"(q.st));  // keeps each group's work where it is written
      __builtin_amdgcn_sched_barrier(0);
    }
    // merge: wave64 butterfly, then the waves in index order through LDS (as in the two-walk kernel)
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      KlState other{__shfl_xor(q.ms, o, kWave), __shfl_xor(q.ss, o, kWave), __shfl_xor(q.us, o, kWave),
                    __shfl_xor(q.mt, o, kWave), __shfl_xor(q.st, o, kWave)};
      merge_kl(q, other);
    }
    int merge_id = tid;
    asm volatile("" : "+v"(merge_id));  // the LDS slot is recomputed per row rather than kept (and spilled)
    const int lane = merge_id & (kWave - 1), w = merge_id / kWave;
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
      const float ls = q.ms * kLn2 + logf(q.ss);
      const float lt = q.mt * kLn2 + logf(q.st);
      const float v = q.us / q.ss - ls + lt;
      kl[row] = v;
      lse_s[row] = ls;
      lse_t[row] = lt;
      bc[0] = -ls * kLog2e;
      bc[1] = gt * (lt - ls - v);
    }
    __syncthreads();
    const float k0 = bc[0], k1 = bc[1];

    // ---- gradient: d = p_s * g * ((x_s - x_t) + lse_t - lse_s - KL), the teacher row a second time (last use:
    // non-temporal), written over the student row in place; the ring slots freed by the last D positions take the first
    // teacher vectors of the next row.
    u32x4* dv = reinterpret_cast<u32x4*>(dstudent + row * stride);
    const u32x4* nsv = reinterpret_cast<const u32x4*>(student + (has_next ? next : row) * stride);
    const u32x4* ntv = reinterpret_cast<const u32x4*>(teacher + (has_next ? next : row) * stride);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));  // recomputed per vector: loop-invariant index registers would not fit
      const int idx = lane_id + j * THREADS;
      launder(srow[j]);
      // one 32-bit word of the vector at a time: a whole vector of both rows unpacked does not fit
      const uint32_t sw[4] = {srow[j].x, srow[j].y, srow[j].z, srow[j].w};
      const uint32_t tw[4] = {ring[j % D].x, ring[j % D].y, ring[j % D].z, ring[j % D].w};
      uint32_t ow[4] = {0u, 0u, 0u, 0u};
      if (!emit_zero) {  // the same answer in every lane of the workgroup: a jump, not a mask
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          float a[VN], b[VN];
          Row<T>::unpack(u32x4{sw[h], 0u, 0u, 0u}, a);
          Row<T>::unpack(u32x4{tw[h], 0u, 0u, 0u}, b);
#pragma unroll
          for (int k = 0; k < VN / 4; ++k) a[k] = fast_exp2(fmaf(a[k], kLog2e, k0)) * fmaf(a[k] - b[k], gt, k1);
          ow[h] = Row<T>::pack(a).x;
          if (h == 1) __builtin_amdgcn_sched_barrier(0);
        }
      }
      srow[j] = u32x4{ow[0], ow[1], ow[2], ow[3]};
      if (j + D < NV) {
        if (has(j + D)) ring[j % D] = load_stream(row_vec(tv, (idx + D * THREADS) * tscale));
      } else {
        ring[j % D] = *row_vec(ntv, lane_id + (j % D) * THREADS);  // the row itself again when there is no next one
      }
      __builtin_amdgcn_sched_barrier(0);  // one vector at a time: hoisting the next one's unpacking spills
    }
    // ---- the gradient out in one burst, the next student row in in one burst
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));
      if (has(j)) store_stream(row_vec(dv, lane_id + j * THREADS), srow[j]);
    }
    // without a next row the row itself is read again, and a lane without a vector at the partial position reads
    // its first vector again (never used): branches here would cost the precise wait counts
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));
      srow[j] = load_stream(row_vec(nsv, has(j) ? lane_id + j * THREADS : lane_id));
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!has_next) return;
    row = next;
  }
}

template <typename T>
struct KlResidentSupported {
  static constexpr bool value = false;
};
template <>
struct KlResidentSupported<bf16_t> {
  static constexpr bool value = true;
};
template <>
struct KlResidentSupported<f16_t> {
  static constexpr bool value = true;
};

template <typename T>
int launch_reverse_kl_resident(const T* student, const T* teacher, int64_t stride, int64_t vocab, int64_t n_rows,
                               const float* g, float grad_scale, float* kl, float* lse_s, float* lse_t, T* dstudent,
                               int compute_units, hipStream_t stream) {
  if constexpr (!KlResidentSupported<T>::value) {
    return RELAX_AMD_EUNSUPPORTED;
  } else {
    constexpr int VN = Row<T>::kPerVec;
    if (vocab % VN != 0) return RELAX_AMD_EUNSUPPORTED;
    const int64_t nvec = vocab / VN;
    const int full = int(nvec / kKlResThreads);
    const bool partial = nvec % kKlResThreads != 0;
    const int64_t blocks = n_rows < compute_units ? n_rows : compute_units;
    const dim3 grid(static_cast<unsigned>(blocks)), block(kKlResThreads);
#define RELAX_AMD_KL_RESIDENT(NVF, PARTIAL)                                                                          \
  if (full == NVF && partial == PARTIAL) {                                                                            \
    hipLaunchKernelGGL((reverse_kl_resident_kernel<T, NVF, PARTIAL>), grid, block, 0, stream, student, teacher,      \
                       stride, vocab, n_rows, g, grad_scale, kl, lse_s, lse_t, dstudent);                            \
    return check_launch("reverse_kl_resident");                                                                      \
  }
    // vocabularies of 151936 / 152064 (18992 / 19008 vectors), 128256 / 129280 (16032 / 16160), 131072 (16384),
    // 100352 / 102400 (12544 / 12800) entries
    RELAX_AMD_KL_RESIDENT(18, true)
    RELAX_AMD_KL_RESIDENT(15, true)
    RELAX_AMD_KL_RESIDENT(16, false)
    RELAX_AMD_KL_RESIDENT(12, true)
#undef RELAX_AMD_KL_RESIDENT
    return RELAX_AMD_EUNSUPPORTED;
  }
}

template int launch_reverse_kl_resident<float>(const float*, const float*, int64_t, int64_t, int64_t, const float*,
                                               float, float*, float*, float*, float*, int, hipStream_t);
template int launch_reverse_kl_resident<bf16_t>(const bf16_t*, const bf16_t*, int64_t, int64_t, int64_t, const float*,
                                                float, float*, float*, float*, bf16_t*, int, hipStream_t);
template int launch_reverse_kl_resident<f16_t>(const f16_t*, const f16_t*, int64_t, int64_t, int64_t, const float*,
                                               float, float*, float*, float*, f16_t*, int, hipStream_t);

}  // namespace relax_amd
