// Fused reverse-KL step with every row shared between eight one-shot workgroups: the same computation and the same
// bits as reverse_kl_step_kernel and reverse_kl_resident_kernel (per-token KL(student || teacher), both log-sum-exps
// and the student gradient for a known d loss / d KL, one launch), in the launch shape this memory system streams
// fastest: many small workgroups that touch their memory once and retire, dispatched in address order.
//
// A row is scanned by 1024 "virtual threads" exactly as reverse_kl_step_kernel lays it out for a 1024-thread workgroup
// (virtual thread t takes the 16-byte vectors t, t + 1024, ... of both rows; two at a time while it has two to go,
// then single ones).  A workgroup here is 128 of those virtual threads (virtual waves 2q and 2q + 1 of the row) and
// holds its share of BOTH rows on chip (2 x 19 vectors per thread at V = 151936: the student's and seven of the
// teacher's in registers, twelve of the teacher's in LDS, where global -> LDS loads put them without a register in
// between; six workgroups per CU), so the student and the teacher row are each read once; the persistent kernel keeps
// the student row and reads the teacher row 1.5 times.  Each wave reduces its share to the five-word state
// of the two online softmaxes by the same butterfly, publishes it, the workgroup's first wave fetches the row's
// sixteen states, merges them in wave order as thread 0 of the 1024-thread workgroup does, and the registers turn
// into the gradient d = p_s * g * ((x_s - x_t) + lse_t - lse_s - KL).
//
// Exchange: the tagged ring of row_exchange.h, a slot of 16 x 5 words per row; a workgroup that gives up its wait
// writes NaN (KL and both log-sum-exps of its row, by the row's first workgroup) instead of hanging.
//
// Replaces, like the other reverse-KL kernels, the jsd_alpha == 0 branch of compute_opd_kl on complete log-softmax rows
// (relax/utils/opd/opd_utils.py:1165-1169) and its autograd backward, for one micro-batch.
//
// hipcc-flags: -mllvm -amdgpu-use-amdgpu-trackers=1
#include "reverse_kl_resident.h"
#include "reverse_kl_math.h"
#include "row_exchange.h"

namespace relax_amd {

constexpr int kKlRowThreads = 1024;                       // virtual threads of a row
constexpr int kKlRowWaves = kKlRowThreads / kWave;        // 16
constexpr int kKlStateWords = 5;                          // KlState
constexpr int kKlSlotWords = kKlRowWaves * kKlStateWords; // 80
constexpr int kKlSplitThreads = 128;
constexpr int kKlSplit = kKlRowThreads / kKlSplitThreads;
constexpr size_t kKlRingWords = size_t(kRing) * kKlSlotWords;

static __device__ __align__(256) unsigned long long kl_split_ring[kKlRingWords + kRingTailWords];

// marks a raw vector as changed without touching it: what is unpacked from it afterwards is a new value to the
// compiler, which would otherwise keep (and spill) the values unpacked earlier for the later uses
__device__ __forceinline__ void kl_split_launder(u32x4& r) {
  asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
}

// absorb_pair() over the values of kKlUnroll raw vector pairs (as absorb_raw_pairs() in reverse_kl_resident.hip: same
// arithmetic, same order)
template <typename T>
__device__ __forceinline__ void kl_split_absorb_raw_pairs(u32x4* s_raw, u32x4* t_raw, KlState& q) {
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
    // unpacked again, one 32-bit word of both vectors at a time: the first walk's values kept alive do not fit the
    // register file next to the two rows
    kl_split_launder(s_raw[u]);
    kl_split_launder(t_raw[u]);
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

// LDS_VECS: the first LDS_VECS teacher vectors of a thread's share go from global memory straight to LDS (16 bytes
// per lane and vector, no register in between) and are read from there by the scan and again by the gradient pass;
// the others and the student's stay in registers.  WAVES_MIN / WAVES_MAX: waves per SIMD the register allocation aims
// for.
template <typename T, int NVF, bool PARTIAL, int LDS_VECS, int WAVES_MIN, int WAVES_MAX>
__global__ __launch_bounds__(kKlSplitThreads) __attribute__((amdgpu_waves_per_eu(WAVES_MIN, WAVES_MAX)))
void reverse_kl_split_kernel(
    const T* __restrict__ student, const T* __restrict__ teacher, int64_t stride, int64_t vocab, int64_t n_rows,
    const float* __restrict__ g, float grad_scale, float* __restrict__ kl, float* __restrict__ lse_s,
    float* __restrict__ lse_t, T* __restrict__ dstudent, unsigned long long* __restrict__ ring, unsigned laps,
    unsigned max_polls, unsigned wait_tag_offset) {
  constexpr int kU = kKlUnroll, ROW_THREADS = kKlRowThreads;
  constexpr int VN = Row<T>::kPerVec;
  constexpr int NV = NVF + (PARTIAL ? 1 : 0);
  constexpr int kGroups = (NV + kU - 1) / kU;
  constexpr int NT = NV - LDS_VECS;  // teacher vectors in registers
  static_assert(LDS_VECS <= NVF && NT >= 1, "only full vector positions go to LDS");
  __shared__ float bc[2];
  __shared__ u32x4 tlds[LDS_VECS > 0 ? LDS_VECS : 1][kKlSplitThreads];
  const int tid = threadIdx.x;
  const bool wave0 = __builtin_amdgcn_readfirstlane(tid) < kWave;
  const unsigned part = blockIdx.x % kKlSplit;
  const int64_t row = blockIdx.x / kKlSplit;
  const int vt = int(part) * kKlSplitThreads + tid;  // virtual thread of the row
  const int rem = int(vocab / VN) - NVF * ROW_THREADS;
  auto has = [&](int j) -> bool { return j < NVF || (PARTIAL && j == NVF && vt < rem); };

  const u32x4* sv = reinterpret_cast<const u32x4*>(student + row * stride);
  const u32x4* tv = reinterpret_cast<const u32x4*>(teacher + row * stride);
  u32x4 sreg[NV], treg[NT];
  {
    const int wave_base = __builtin_amdgcn_readfirstlane(tid / kWave) * kWave;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      if (has(j)) sreg[j] = load_stream(sv + vt + j * ROW_THREADS);
      if (j < LDS_VECS)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(tv + vt + j * ROW_THREADS),
                                         (__attribute__((address_space(3))) void*)(&tlds[j][wave_base]), 16, 0, 0);
      else if (has(j))
        treg[j - LDS_VECS] = load_stream(tv + vt + j * ROW_THREADS);
    }
  }
  // teacher vector j of this thread
  auto teacher_vec = [&](int j) -> u32x4 { return j < LDS_VECS ? tlds[j < LDS_VECS ? j : 0][tid] : treg[j < LDS_VECS ? 0 : j - LDS_VECS]; };
  unsigned* status = reinterpret_cast<unsigned*>(ring + kKlRingWords);
  const unsigned tag = exchange_tag(status, laps, row);
  const float gt = g[row] * grad_scale;

  // the scan, pair by pair as the vectors arrive, in reverse_kl_step_kernel's order
  KlState q{kNegHuge, 0.f, 0.f, kNegHuge, 0.f};
  bool grouped = true;
#pragma unroll
  for (int gi = 0; gi < kGroups; ++gi) {
    const int j0 = kU * gi, j1 = kU * gi + 1;
    if (grouped && j1 < NV && has(j1)) {
      u32x4 tpair[kU] = {teacher_vec(j0), teacher_vec(j1 < NV ? j1 : 0)};
      kl_split_absorb_raw_pairs<T>(&sreg[j0 < NV - 1 ? j0 : 0], tpair, q);
    } else {
      grouped = false;
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (j0 + u < NV && has(j0 + u)) {
          float a[VN], b[VN];
          Row<T>::unpack(sreg[j0 + u < NV ? j0 + u : NV - 1], a);
          Row<T>::unpack(teacher_vec(j0 + u < NV ? j0 + u : NV - 1), b);
          absorb_pair(a, b, q);
        }
    }
    asm volatile("" : "+v"(q.ss), "+v"(q.us), "+v"(q.st));  // keeps each group's work where it is written
    __builtin_amdgcn_sched_barrier(0);
  }
  // each wave to its state (the first half of the 1024-thread workgroup's merge); lane 0's copy is the one that
  // counts (the butterfly's merge is not symmetric in its last bits), published by lanes 0..4
  wave_butterfly([&](auto o) {
    constexpr int O = decltype(o)::value;
    KlState other{lane_xor<O>(q.ms), lane_xor<O>(q.ss), lane_xor<O>(q.us), lane_xor<O>(q.mt), lane_xor<O>(q.st)};
    merge_kl(q, other);
  });
  unsigned long long* slot = ring + size_t(row % kRing) * kKlSlotWords;
  {
    const float w0 = lane_value(q.ms), w1 = lane_value(q.ss), w2 = lane_value(q.us), w3 = lane_value(q.mt),
                w4 = lane_value(q.st);
    const int lane = vt & (kWave - 1), vwave = vt / kWave;
    if (lane < kKlStateWords) {
      const float val = lane == 0 ? w0 : lane == 1 ? w1 : lane == 2 ? w2 : lane == 3 ? w3 : w4;
      exchange_store(slot + vwave * kKlStateWords + lane, tag, val);
    }
  }

  if (wave0) {
    // lanes 0..63 fetch the slot's words 0..63, lanes 0..15 also words 64..79; then every lane merges the sixteen
    // states in wave order
    __builtin_amdgcn_s_setprio(3);
    float lo = 0.f, hi = 0.f;
    bool gave_up = !exchange_wait(slot + tid, tag + wait_tag_offset, max_polls, status, lo);
    if (tid < kKlSlotWords - kWave && !gave_up)
      gave_up = !exchange_wait(slot + kWave + tid, tag + wait_tag_offset, max_polls, status, hi);
    const bool any_gave_up = __any(gave_up);
    if (any_gave_up && tid == 0) exchange_report_give_up(status);
    auto word = [&](int i) {  // word i of the slot, in every lane
      return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(i < kWave ? lo : hi), i & (kWave - 1)));
    };
    KlState whole{word(0), word(1), word(2), word(3), word(4)};
#pragma unroll
    for (int i = 1; i < kKlRowWaves; ++i) {
      const KlState other{word(5 * i), word(5 * i + 1), word(5 * i + 2), word(5 * i + 3), word(5 * i + 4)};
      merge_kl(whole, other);
    }
    KlRow r = kl_finish(whole);
    if (any_gave_up) r.kl = r.lse_s = r.lse_t = __builtin_nanf("");
    if (tid == 0) {
      if (part == 0) {
        kl[row] = r.kl;
        lse_s[row] = r.lse_s;
        lse_t[row] = r.lse_t;
      }
      bc[0] = -r.lse_s * kLog2e;
      bc[1] = gt * (r.lse_t - r.lse_s - r.kl);
    }
    __builtin_amdgcn_s_setprio(0);
  }
  __syncthreads();
  const float k0 = bc[0], k1 = bc[1];
  u32x4* dv = reinterpret_cast<u32x4*>(dstudent + row * stride);
  if (gt == 0.f) {  // uniform over the workgroup: a token without gradient gets a zero row
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (has(j)) store_stream(dv + vt + j * ROW_THREADS, u32x4{0u, 0u, 0u, 0u});
    return;
  }
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    int lane_id = vt;
    asm volatile("" : "+v"(lane_id));
    kl_split_launder(sreg[j]);
    u32x4 tvec = teacher_vec(j);
    kl_split_launder(tvec);
    // one 32-bit word of the two vectors at a time
    const uint32_t sw[4] = {sreg[j].x, sreg[j].y, sreg[j].z, sreg[j].w};
    const uint32_t tw[4] = {tvec.x, tvec.y, tvec.z, tvec.w};
    uint32_t ow[4];
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
    if (has(j)) store_stream(dv + lane_id + j * ROW_THREADS, u32x4{ow[0], ow[1], ow[2], ow[3]});
    __builtin_amdgcn_sched_barrier(0);
  }
}

namespace {
ExchangeRingCache kl_ring_cache;
}

// Long rows (12 and more vector positions per thread): three waves per SIMD, i.e. six workgroups per CU, each with
// twelve teacher vectors per thread (24 KB) in LDS; with both rows in registers only two waves per SIMD fit, which is
// 9 % slower on 16384 x 151936 rows (2.71 - 2.73 against 2.47 ms).  Shorter rows fit the registers of four and more
// waves per SIMD as they are.  Rows of more than 20 vectors per thread (vocabularies of 200 k - 262 k entries): two
// waves per SIMD (256 registers a lane, four workgroups per CU) with eighteen teacher vectors per thread (36 KB) in LDS.
template <int NVF>
constexpr int kl_split_lds_vecs() {
  return NVF >= 24 ? 18 : NVF >= 12 ? 12 : 0;
}
template <int NVF>
constexpr int kl_split_waves_min() {
  return NVF >= 24 ? 2 : NVF >= 12 ? 3 : 4;
}
template <int NVF>
constexpr int kl_split_waves_max() {
  return NVF >= 24 ? 2 : NVF >= 12 ? 3 : 8;
}

template <typename T>
struct KlSplitSupported {
  static constexpr bool value = false;
};
template <>
struct KlSplitSupported<bf16_t> {
  static constexpr bool value = true;
};
template <>
struct KlSplitSupported<f16_t> {
  static constexpr bool value = true;
};

template <typename T>
int launch_reverse_kl_split(const T* student, const T* teacher, int64_t stride, int64_t vocab, int64_t n_rows,
                            const float* g, float grad_scale, float* kl, float* lse_s, float* lse_t, T* dstudent,
                            hipStream_t stream) {
  if constexpr (!KlSplitSupported<T>::value) {
    return RELAX_AMD_EUNSUPPORTED;
  } else {
    constexpr int VN = Row<T>::kPerVec;
    if (vocab % VN != 0 || n_rows * kKlSplit > 2147483647LL) return RELAX_AMD_EUNSUPPORTED;
    const int64_t nvec = vocab / VN;
    const int full = int(nvec / kKlRowThreads);
    const bool partial = nvec % kKlRowThreads != 0;
    // the row shapes launch_reverse_kl_resident is built for, and rows of 6145 .. 8192 vectors (50304, 64000 / 65536
    // entries: 1.91 / 2.33 / 2.08 ms on 32768 rows where the two-walk kernel takes 2.11 / 2.79 / 2.74).  Rows of
    // 32000 entries, four vectors per thread, are left to the two-walk kernel: here the exchange outweighs the second
    // read (2.77 against 2.52 ms on 65536 rows).
    if (!((full == 24 && partial) || (full == 30 && partial) || (full == 31 && partial) || (full == 32 && !partial) ||
          (full == 20 && !partial) || (full == 19 && partial) || (full == 18 && partial) || (full == 15 && partial) ||
          (full == 16 && !partial) || (full == 12 && partial) || (full == 8 && !partial) || (full == 7 && partial) ||
          (full == 6 && partial)))
      return RELAX_AMD_EUNSUPPORTED;
    unsigned long long* ring = nullptr;
    if (int rc = exchange_ring_of_device(kl_ring_cache, reinterpret_cast<const void*>(&kl_split_ring),
                                         "reverse_kl_split", &ring))
      return rc;
    const unsigned laps = unsigned((n_rows + kRing - 1) / kRing);
    const unsigned max_polls = exchange_max_polls();
    const unsigned tag_offset = exchange_wait_tag_offset();
    hipLaunchKernelGGL(exchange_ring_advance_kernel<kKlRingWords>, dim3(1), dim3(256), 0, stream, ring, laps,
                       static_cast<unsigned long long*>(nullptr), size_t(0));
    const dim3 grid(static_cast<unsigned>(n_rows * kKlSplit)), block(kKlSplitThreads);
#define RELAX_AMD_KL_SPLIT(NVF, PARTIAL)                                                                              \
  if (full == NVF && partial == PARTIAL) {                                                                            \
    hipLaunchKernelGGL((reverse_kl_split_kernel<T, NVF, PARTIAL, kl_split_lds_vecs<NVF>(), kl_split_waves_min<NVF>(), \
                                                kl_split_waves_max<NVF>()>),                                          \
                       grid, block, 0, stream, student, teacher, stride, vocab, n_rows, g, grad_scale, kl, lse_s,    \
                       lse_t, dstudent, ring, laps, max_polls, tag_offset);                                           \
    return check_launch("reverse_kl_split");                                                                          \
  }
    // 200064 / 201088 / 202048, 248320 / 250880, 256000, 262144 entries
    RELAX_AMD_KL_SPLIT(24, true)
    RELAX_AMD_KL_SPLIT(30, true)
    RELAX_AMD_KL_SPLIT(31, true)
    RELAX_AMD_KL_SPLIT(32, false)
    RELAX_AMD_KL_SPLIT(20, false)
    RELAX_AMD_KL_SPLIT(19, true)
    RELAX_AMD_KL_SPLIT(18, true)
    RELAX_AMD_KL_SPLIT(15, true)
    RELAX_AMD_KL_SPLIT(16, false)
    RELAX_AMD_KL_SPLIT(12, true)
    RELAX_AMD_KL_SPLIT(8, false)
    RELAX_AMD_KL_SPLIT(7, true)
    RELAX_AMD_KL_SPLIT(6, true)
#undef RELAX_AMD_KL_SPLIT
    return RELAX_AMD_EUNSUPPORTED;
  }
}

template int launch_reverse_kl_split<float>(const float*, const float*, int64_t, int64_t, int64_t, const float*, float,
                                            float*, float*, float*, float*, hipStream_t);
template int launch_reverse_kl_split<bf16_t>(const bf16_t*, const bf16_t*, int64_t, int64_t, int64_t, const float*,
                                             float, float*, float*, float*, bf16_t*, hipStream_t);
template int launch_reverse_kl_split<f16_t>(const f16_t*, const f16_t*, int64_t, int64_t, int64_t, const float*, float,
                                            float*, float*, float*, f16_t*, hipStream_t);

}  // namespace relax_amd
