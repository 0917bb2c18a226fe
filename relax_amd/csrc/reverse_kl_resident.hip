// Register-resident fused reverse-KL step: the same computation as reverse_kl_step_kernel (per-token
// KL(student || teacher), both log-sum-exps and the student gradient for a known d loss / d KL, one launch) for long
// 16-bit rows of the common vocabulary sizes.
//
// A 1024-thread workgroup keeps the STUDENT row in its vector registers (19 16-byte vectors per thread at
// V = 151936) and streams the teacher row past it twice: once for the two online softmaxes, once for the gradient
// d = p_s * g * ((x_s - x_t) + lse_t - lse_s - KL).  HBM sees the student row once instead of twice (the two-walk
// kernel re-fetches ~85 % of both rows through the fabric).  The teacher row passes through eight slots of LDS (one
// 16-byte vector per thread each, 128 KB), filled by loads that go from global memory straight to LDS: up to eight
// vectors per thread are in flight ahead of their use without a register being held for them, and since the scan ends
// with the row's last eight vectors in the slots, the gradient pass walks the row backwards and reads only the other
// NV - 8 again.  Workgroups are persistent, one per CU, rows b, b + grid, ...; a row's gradient replaces the student
// row in the registers, leaves in one burst of stores, and the workgroup's next student row arrives in one burst of
// loads, which the next scan lets land completely before it starts.  On 16384 x 151936 rows: 2.97 ms with a register
// ring of four teacher vectors and the gradient stored / the next row loaded vector by vector behind the arithmetic,
// 2.84 ms with the two bursts, 2.75 ms with the LDS slots (and 2.78 ms when the scan starts on the first vectors of
// the arriving burst instead of waiting for all of it: memory rewards requests of one kind in long runs).  No
// workgroup waits for another; the loop bound is the only exit condition.
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
// Teacher vectors in flight ahead of their use, or kept for the second pass: slots of one 16-byte vector per thread in
// LDS (128 KB of the CU's 160), filled by loads that go from global memory straight to LDS and cost no registers.
constexpr int kKlSlots = 8;

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

// This thread's 16 bytes of an LDS slot once the request that fills them has arrived: vector-memory operations complete
// in the order they were issued, so "at most VM still in flight" says it has, VM being the number of operations this
// wave is known to have issued after it.  The wait and the read are one opaque statement because the compiler's own
// bookkeeping of loads that land in LDS only knows "all of them": it would wait for every request in flight, the ones
// issued a moment ago included, in front of every read.
template <int VM>
__device__ __forceinline__ u32x4 lds_read_when_at_most(uint32_t lds_byte_address) {
  u32x4 r;
  asm volatile("s_waitcnt vmcnt(%2)\n\tds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)"
               : "=v"(r)
               : "v"(lds_byte_address), "n"(VM)
               : "memory");
  return r;
}
// the largest wait count <= in_flight_after that has an instantiation (in_flight_after folds to a constant where the
// loops around the call are unrolled)
template <int N>
struct SlotRead {
  static __device__ __forceinline__ u32x4 go(uint32_t a, int in_flight_after) {
    return in_flight_after >= N ? lds_read_when_at_most<N>(a) : SlotRead<N - 1>::go(a, in_flight_after);
  }
};
template <>
struct SlotRead<0> {
  static __device__ __forceinline__ u32x4 go(uint32_t a, int) { return lds_read_when_at_most<0>(a); }
};

template <typename T>
__device__ __forceinline__ void absorb_raw_pairs(u32x4* s_raw, u32x4* t_raw, KlState& q) {
  constexpr int VN = Row<T>::kPerVec;
  float smax = 0.f, tmax = 0.f;
#pragma unroll
  for (int u = 0; u < kKlUnroll; ++u) {
    float a[VN], b[VN];
    Row<T>::unpack(s_raw[u], a);
    Row<T>::unpack(t_raw[u], b);
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
    launder(t_raw[u]);
    // one 32-bit word of the vectors at a time, in element order
    const uint32_t sw[4] = {s_raw[u].x, s_raw[u].y, s_raw[u].z, s_raw[u].w};
    const uint32_t tw[4] = {t_raw[u].x, t_raw[u].y, t_raw[u].z, t_raw[u].w};
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
  constexpr int THREADS = kKlResThreads, kU = kKlUnroll, S = kKlSlots;
  constexpr int VN = Row<T>::kPerVec;
  constexpr int NV = NVF + (PARTIAL ? 1 : 0);  // vector positions per thread
  constexpr int kGroups = (NV + kU - 1) / kU;
  static_assert(kU == 2 && NV > S && S % kU == 0, "the teacher slots are refilled pair by pair");
  __shared__ float lds[THREADS / kWave][5];
  __shared__ float bc[2];
  // one object per slot: reads of one slot can then be told apart from the loads in flight into the others
  __shared__ u32x4 slot0[THREADS], slot1[THREADS], slot2[THREADS], slot3[THREADS], slot4[THREADS], slot5[THREADS],
      slot6[THREADS], slot7[THREADS];
  const int tid = threadIdx.x;
  const int rem = int(vocab / VN) - NVF * THREADS;  // lanes that hold a vector at the partial position (host-checked)
  u32x4 srow[NV];  // the student row

  // does this lane hold a vector at position j?  A compile-time answer except at the partial position.
  auto has = [&](int j) -> bool { return j < NVF || (PARTIAL && j == NVF && tid < rem); };
  auto slot = [&](int k) -> u32x4* {
    switch (k) {
      case 0: return slot0;
      case 1: return slot1;
      case 2: return slot2;
      case 3: return slot3;
      case 4: return slot4;
      case 5: return slot5;
      case 6: return slot6;
      default: return slot7;
    }
  };
  // teacher vector j of the row at `base` -> slot j % S, this thread's 16 bytes of it; global memory to LDS without a
  // register in between.  A lane without a vector at the partial position requests its first vector again (never
  // used): the request is issued by every wave, which keeps the count of requests in flight the same for all.
  auto request = [&](const u32x4* base, int j, uint32_t scale) {
    int lane_id = tid;
    asm volatile("" : "+v"(lane_id));  // recomputed per request: loop-invariant index registers would not fit
    const uint32_t index = uint32_t(has(j) ? lane_id + j * THREADS : lane_id) * scale;
    const int wave = __builtin_amdgcn_readfirstlane(lane_id / kWave);
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(row_vec(base, index)),
                                     (__attribute__((address_space(3))) void*)(slot(j % S) + wave * kWave), 16, 0, 0);
  };

  // the slot of teacher vector j, valid once at most `in_flight_after` of this wave's later vector-memory operations
  // are outstanding
  auto teacher_vec = [&](int j, int in_flight_after) -> u32x4 {
    int lane_id = tid;
    asm volatile("" : "+v"(lane_id));
    const uint32_t a = uint32_t(uintptr_t((__attribute__((address_space(3))) u32x4*)(slot(j % S) + lane_id)));
    // the counts that occur: NV or more ahead of the scan's own requests, fewer than S behind them
    return in_flight_after >= NV ? lds_read_when_at_most<NV>(a) : SlotRead<S - 1>::go(a, in_flight_after);
  };

  int64_t row = blockIdx.x;
  if (row >= n_rows) return;
  {
    // the first S teacher vectors, last first (as every later row finds them requested by its predecessor), then the
    // student row
    const u32x4* tv0 = reinterpret_cast<const u32x4*>(teacher + row * stride);
#pragma unroll
    for (int j = S - 1; j >= 0; --j) request(tv0, j, 1u);
    const u32x4* sv = reinterpret_cast<const u32x4*>(student + row * stride);
#pragma unroll
    for (int j = 0; j < NV; ++j) srow[j] = load_stream(row_vec(sv, has(j) ? tid + j * THREADS : tid));
  }

  while (true) {
    const int64_t next = row + gridDim.x;
    const bool has_next = next < n_rows;
    const float gt = g[row] * grad_scale;
    const u32x4* tv = reinterpret_cast<const u32x4*>(teacher + row * stride);

    // a token without gradient (g == 0) gets a zero row; the second pass's teacher requests then all go to the row's
    // first vector, which costs nothing, so that the instruction stream -- and with it the wait counts -- stays the same
    const bool emit_zero = gt == 0.f;
    const uint32_t tscale = emit_zero ? 0u : 1u;

    // ---- scan: both online softmaxes and sum e_s * (x_s - x_t).  The teacher row streams through the S slots: its
    // first S vectors are already on their way (requested during the previous row's gradient pass), a slot just read
    // takes the vector S positions further on, and the pass ends with the row's last S vectors in LDS.
    KlState q{kNegHuge, 0.f, 0.f, kNegHuge, 0.f};
    bool grouped = true;
    // The whole student row first (vmcnt = 0, the other counters left alone): a scan that starts on the first vectors
    // of the arriving burst mixes its own teacher requests into it and measured slower (2.78 against 2.75 ms).
    __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
    for (int gi = 0; gi < kGroups; ++gi) {
      const int j0 = kU * gi, j1 = kU * gi + 1;
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));
      // Requests of this wave issued after the one that filled the slot of vector j, at the least: for the first S
      // vectors (requested during the previous row's gradient pass, or ahead of the first row) the NV loads of the
      // student row and this scan's own requests so far; for the others the scan's requests that followed theirs.
      constexpr int kScanRequests = NV - S;
      const int issued = kU * gi < kScanRequests ? kU * gi : kScanRequests;  // by the groups before this one
      auto after = [&](int j) -> int { return j < S ? NV + issued : issued - (j - S) - 1; };
      if (grouped && j1 < NV && has(j1)) {
        u32x4 tpair[kU] = {teacher_vec(j0, after(j1)), teacher_vec(j1, after(j1))};
        absorb_raw_pairs<T>(&srow[j0 < NV - 1 ? j0 : 0], tpair, q);
      } else {
        grouped = false;
#pragma unroll
        for (int u = 0; u < kU; ++u)
          if (j0 + u < NV && has(j0 + u)) {
            float a[VN], b[VN];
            launder(srow[j0 + u < NV ? j0 + u : NV - 1]);
            Row<T>::unpack(srow[j0 + u < NV ? j0 + u : NV - 1], a);
            Row<T>::unpack(teacher_vec(j0 + u, after(j0 + u)), b);
            absorb_pair(a, b, q);
          }
      }
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (j0 + u + S < NV) request(tv, j0 + u + S, 1u);
      asm volatile("" : "+v"(q.ss), "+v"(q.us), "+v"(q.st));  // keeps each group's work where it is written
      __builtin_amdgcn_sched_barrier(0);
    }
    // merge: wave64 butterfly, then the waves in index order through LDS (as in the two-walk kernel)
    wave_butterfly([&](auto o) {
      constexpr int O = decltype(o)::value;
      KlState other{lane_xor<O>(q.ms), lane_xor<O>(q.ss), lane_xor<O>(q.us), lane_xor<O>(q.mt), lane_xor<O>(q.st)};
      merge_kl(q, other);
    });
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
      const KlRow r = kl_finish(q);
      const float ls = r.lse_s, lt = r.lse_t, v = r.kl;
      kl[row] = v;
      lse_s[row] = ls;
      lse_t[row] = lt;
      bc[0] = -ls * kLog2e;
      bc[1] = gt * (lt - ls - v);
    }
    __syncthreads();
    const float k0 = bc[0], k1 = bc[1];

    // ---- gradient: d = p_s * g * ((x_s - x_t) + lse_t - lse_s - KL), written over the student row in place, from the
    // row's end to its beginning: the last S teacher vectors are still in LDS, each slot read takes the vector S
    // positions further down (the teacher's second read: only NV - S of its NV vectors), and the slots of the first
    // S positions take the first teacher vectors of the next row.
    const u32x4* ntv = reinterpret_cast<const u32x4*>(teacher + (has_next ? next : row) * stride);
#pragma unroll
    for (int j = NV - 1; j >= 0; --j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));
      launder(srow[j]);
      // the last S vectors have been in LDS since the scan; the others were requested S steps ago, S - 1 requests
      // (one per step) followed theirs
      const u32x4 tvec = teacher_vec(j, NV - 1 - j < S - 1 ? NV - 1 - j : S - 1);
      // one 32-bit word of the vector at a time: a whole vector of both rows unpacked does not fit
      const uint32_t sw[4] = {srow[j].x, srow[j].y, srow[j].z, srow[j].w};
      const uint32_t tw[4] = {tvec.x, tvec.y, tvec.z, tvec.w};
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
      if (j >= S)
        request(tv, j - S, tscale);
      else
        request(ntv, j, 1u);  // the row itself again when there is no next one
      __builtin_amdgcn_sched_barrier(0);  // one vector at a time: hoisting the next one's unpacking spills
    }
    // ---- the gradient out in one burst, the next student row in in one burst
    u32x4* dv = reinterpret_cast<u32x4*>(dstudent + row * stride);
    const u32x4* nsv = reinterpret_cast<const u32x4*>(student + (has_next ? next : row) * stride);
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
    // vocabularies of 163840 (20480 vectors) and up to it, 151936 / 152064 (18992 / 19008), 128256 / 129280
    // (16032 / 16160), 131072 (16384),
    // 100352 / 102400 (12544 / 12800) entries
    RELAX_AMD_KL_RESIDENT(20, false)
    RELAX_AMD_KL_RESIDENT(19, true)
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
