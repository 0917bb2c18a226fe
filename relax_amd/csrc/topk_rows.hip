// Row-wise top-K selection over the vocabulary: the K largest logits of every response row and their vocabulary ids,
// sorted by value (largest first).  Replaces ``torch.topk(logits_chunk, k=k, dim=-1)`` in get_log_probs_and_entropy
// (relax/backends/megatron/loss.py:434-436), which the actor runs over every response row when it collects the
// student's top-K ids for on-policy distillation (relax/backends/megatron/actor.py:651-653).
//
// One 1024-thread workgroup per row, working on order-preserving 32-bit keys of the fp32 values.  Usually a shortcut
// suffices: the k-th largest of the 1024 per-thread maxima is a lower bound of the row's k-th largest value, the few
// hundred elements at or above (the 12-bit bin of) that bound are collected in a second look that skips every group
// of eight vectors whose maximum, noted during the first look, lies below the bound, and are ranked in LDS.  Rows where
// that leaves too many candidates (long runs of equal or nearly equal values) take the general way, a radix select:
//   1. histogram of the keys' leading 12 bits (wave-private 16-bit counters in LDS, so that a wave's atomics only
//      meet that wave's own conflicts), totals per bin, a workgroup-wide suffix scan from the top bin down: the bin
//      that holds the K-th largest key, how many keys lie above it and how many inside;
//   2. while that bin holds more keys than the list has room for (rows with long runs of equal or nearly equal
//      values), the same again on the next 12 bits of the keys that share the prefix found so far;
//   3. one more pass over the row collects (key, index) of everything above the final prefix plus the keys that share
//      it (at most kTkCap of them; with every bit consumed they are exact ties and any of them will do);
//   4. that short list is ordered in LDS (key descending, then index ascending: by counting ranks up to 512 entries,
//      by a bitonic sort beyond); the first K entries leave.
// NaN orders above +inf (as torch.topk does); -0 orders below +0; which of several equal
// values at the threshold is taken is unspecified in torch as well -- here the list order decides.
#include "device_utils.h"
#include "relax_amd.h"
#include "row_scan.h"

namespace relax_amd {

constexpr int kTkThreads = 1024, kTkWaves = kTkThreads / kWave;
constexpr int kTkDigitBits = 12, kTkBins = 1 << kTkDigitBits;
constexpr int kTkCap = 4096;   // keys sharing the final prefix that are kept for the sort
constexpr int kTkMaxK = 512;
constexpr int kTkList = 8192;  // >= kTkMaxK + kTkCap entries, a power of two
constexpr int kTkRankMax = 512;  // lists up to this length are ranked by counting instead of sorted
static_assert(kTkList >= kTkMaxK + kTkCap && (kTkList & (kTkList - 1)) == 0, "list capacity");
static_assert(kTkList * 8 <= kTkWaves * kTkBins * 2, "the list reuses the histogram's memory");
static_assert(kTkBins == 4 * kTkThreads, "the suffix scan gives every thread four bins");

__device__ __forceinline__ uint32_t tk_key(float v) {
  if (v != v) return 0xFFFFFFFFu;
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float tk_value(uint32_t key) {
  if (key == 0xFFFFFFFFu) return __builtin_nanf("");
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
}

// f(index, value) for every element of the row: 16-byte loads where the row allows them, kTkBatch of them in flight
// per thread (one workgroup per CU has to cover the memory latency by itself); LAST marks the row's last reading
constexpr int kTkBatch = 8;
template <typename T, bool VEC, bool LAST, typename F>
__device__ __forceinline__ void tk_for_each(const T* __restrict__ x, int64_t vocab, F&& f) {
  constexpr int VN = Row<T>::kPerVec;
  const int64_t nvec = VEC ? vocab / VN : 0;
  if (VEC) {
    const u32x4* xv = reinterpret_cast<const u32x4*>(x);
    for (int64_t i0 = threadIdx.x; i0 < nvec; i0 += int64_t(kTkBatch) * kTkThreads) {
      u32x4 raw[kTkBatch];
#pragma unroll
      for (int u = 0; u < kTkBatch; ++u) {
        const int64_t i = i0 + int64_t(u) * kTkThreads;
        if (i < nvec) raw[u] = LAST ? load_stream(xv + i) : xv[i];
      }
#pragma unroll
      for (int u = 0; u < kTkBatch; ++u) {
        const int64_t i = i0 + int64_t(u) * kTkThreads;
        if (i < nvec) {
          float v[VN];
          Row<T>::unpack(raw[u], v);
#pragma unroll
          for (int k = 0; k < VN; ++k) f(uint32_t(i * VN + k), v[k]);
        }
      }
    }
  }
  for (int64_t e = nvec * VN + threadIdx.x; e < vocab; e += kTkThreads) f(uint32_t(e), Row<T>::load1(x + e));
}

// tot[] holds bin counts (complete and visible to the workgroup): finds, from the top bin down, the bin with the
// `wanted`-th key and leaves (bin, keys above it, keys inside it) in found[]; thread t owns bins 4095 - 4t - j, j = 0..3.
// The counted keys must be at least `wanted`, and wanted >= 1.
__device__ __forceinline__ void tk_locate(const uint32_t* tot, uint32_t* wave_part, uint32_t* found, uint32_t wanted) {
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  uint32_t own[4], mine = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    own[j] = tot[kTkBins - 1 - 4 * tid - j];
    mine += own[j];
  }
  uint32_t incl = mine;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t up = __shfl_up(incl, o, kWave);
    if (lane >= o) incl += up;
  }
  if (lane == kWave - 1) wave_part[wave] = incl;
  __syncthreads();
  for (int w = 0; w < wave; ++w) incl += wave_part[w];
  const uint32_t excl = incl - mine;
  if (incl >= wanted && excl < wanted) {  // exactly one thread
    uint32_t above = excl;
    int j = 0;
    while (j < 3 && above + own[j] < wanted) above += own[j++];
    found[0] = uint32_t(kTkBins - 1 - 4 * tid - j);
    found[1] = above;
    found[2] = own[j];
  }
  __syncthreads();
}

// list[0 .. len) holds (key << 32 | ~index) of every element of the top k and not many more (complete and visible):
// bitonic sort, key descending then index ascending, and the first k entries leave.  `capacity` is a power of two.
__device__ __forceinline__ void tk_sort_emit(uint64_t* list, uint32_t len, uint32_t capacity, int k, int64_t tok,
                                             float* __restrict__ out_values, int64_t* __restrict__ out_indices,
                                             uint32_t* rank) {
  const uint32_t tid = threadIdx.x;
  if (len > capacity) len = capacity;
  uint32_t padded = 2;
  while (padded < len) padded <<= 1;
  if (padded <= uint32_t(kTkRankMax)) {
    // a short list (the usual case) is ranked instead of sorted: an entry's place is the number of entries above it
    // (entries are distinct: the index is part of them).  The 1024 threads split the len^2 comparisons, `padded`
    // entries by 1024 / padded stretches of the list; three barriers instead of dozens.
    const uint32_t stretches = kTkThreads / padded, mine = tid % padded, part = tid / padded;
    if (tid < uint32_t(kTkRankMax)) rank[tid] = 0u;
    __syncthreads();
    if (mine < len) {
      const uint64_t me = list[mine];
      const uint32_t per = (len + stretches - 1) / stretches;
      const uint32_t begin = part * per, end = begin + per < len ? begin + per : len;
      uint32_t above = 0;
      for (uint32_t i = begin; i < end; ++i) above += list[i] > me ? 1u : 0u;
      if (above) atomicAdd(&rank[mine], above);
    }
    __syncthreads();
    if (tid < len && rank[tid] < uint32_t(k)) {
      const uint64_t entry = list[tid];
      const uint32_t at = rank[tid];
      out_indices[tok * k + at] = int64_t(0xFFFFFFFFu - uint32_t(entry));
      if (out_values) out_values[tok * k + at] = tk_value(uint32_t(entry >> 32));
    }
    return;
  }
  for (uint32_t i = len + tid; i < padded; i += kTkThreads) list[i] = 0ull;  // below every real entry
  __syncthreads();
  for (uint32_t span = 2; span <= padded; span <<= 1)
    for (uint32_t j = span >> 1; j > 0; j >>= 1) {
      for (uint32_t t = tid; t < padded / 2; t += kTkThreads) {
        const uint32_t i = ((t & ~(j - 1)) << 1) | (t & (j - 1));
        const uint32_t l = i | j;
        const uint64_t a = list[i], b = list[l];
        const bool descending = (i & span) == 0;
        if (descending ? a < b : a > b) {
          list[i] = b;
          list[l] = a;
        }
      }
      __syncthreads();
    }
  for (uint32_t t = tid; t < uint32_t(k); t += kTkThreads) {
    const uint64_t entry = list[t];
    out_indices[tok * k + t] = int64_t(0xFFFFFFFFu - uint32_t(entry));
    if (out_values) out_values[tok * k + t] = tk_value(uint32_t(entry >> 32));
  }
}

// The shortcut, one workgroup per row, two workgroups per CU (32 KB of LDS each).  Every thread's largest key is an
// element of the row, so the row has at least k elements that are >= the k-th largest of the 1024 thread maxima:
// whatever lies below the bin of that maximum cannot be among the top k.  Usually a few hundred elements remain; they
// are collected in a second pass and sorted.  A row that leaves more than the list holds is flagged for the general
// kernel instead.
constexpr int kTkFastList = 2048;
constexpr int kTkFastBatch = 6;  // loads in flight per thread within 64 registers (two workgroups per CU)
constexpr int kTkGroups = 8192;  // groups of eight vectors the shortcut keeps a maximum for (vocab <= 524288 at 16 bit)
// The shortcut's bound, shared by the selection kernel and the fused log-prob + selection kernel: `best` is each
// thread's largest key.  Finds the k-th largest of the thread maxima (at most the 1024-th) to 24 bits -- the 12-bit bin
// that holds it, then the 12-bit sub-bin inside that bin -- and returns the lower end of that sub-bin as a float:
// !(v < bound) holds for every value whose key is at or above it (and for NaN, and for -0 against a bound of +0: a
// few candidates more never hurt).  The first 12 bits alone (sign, exponent, three mantissa bits) would put the bound
// up to an eighth below the value and triple the candidates of a Gaussian row.  *floor_key receives the bound as a
// key; *count is cleared for the collection that follows.
__device__ __forceinline__ float tk_fast_floor(uint32_t best, int k, uint32_t* tot, uint32_t* wave_part,
                                               uint32_t* found, uint32_t* count, uint32_t* floor_key) {
  const int tid = threadIdx.x;
  const uint32_t wanted = uint32_t(k) < uint32_t(kTkThreads) ? uint32_t(k) : uint32_t(kTkThreads);
  for (int d = tid; d < kTkBins; d += kTkThreads) tot[d] = 0u;
  if (tid == 0) *count = 0u;
  __syncthreads();
  atomicAdd(&tot[best >> (32 - kTkDigitBits)], 1u);
  __syncthreads();
  tk_locate(tot, wave_part, found, wanted);
  const uint32_t bin = found[0], still = wanted - found[1];  // the still-th largest inside the bin is the one
  __syncthreads();  // everyone has read found[] and tot[]
  for (int d = tid; d < kTkBins; d += kTkThreads) tot[d] = 0u;
  __syncthreads();
  if ((best >> (32 - kTkDigitBits)) == bin) atomicAdd(&tot[(best >> (32 - 2 * kTkDigitBits)) & (kTkBins - 1)], 1u);
  __syncthreads();
  tk_locate(tot, wave_part, found, still);
  const uint32_t key = (bin << (32 - kTkDigitBits)) | (found[0] << (32 - 2 * kTkDigitBits));
  *floor_key = key;
  return tk_value(key);
}

// One candidate of the shortcut's second look: kept when it is not below the bound.
__device__ __forceinline__ void tk_fast_consider(uint32_t idx, float v, float floor_value, uint64_t* list,
                                                 uint32_t* count) {
  if (!(v < floor_value)) {
    const uint32_t key = tk_key(v);
    const uint32_t slot = atomicAdd(count, 1u);
    if (slot < uint32_t(kTkFastList)) list[slot] = (uint64_t(key) << 32) | uint64_t(0xFFFFFFFFu - idx);
  }
}

// After the second look: ranks the candidates and emits the first k, or flags the row for the general kernel when the
// candidates did not fit the list.
__device__ __forceinline__ void tk_fast_finish(uint64_t* list, const uint32_t* count, int k, int64_t tok,
                                               float* __restrict__ out_values, int64_t* __restrict__ out_indices,
                                               uint8_t* __restrict__ needs_general, uint32_t* rank) {
  __syncthreads();
  const uint32_t len = *count;
  if (threadIdx.x == 0) needs_general[tok] = len > uint32_t(kTkFastList) ? 1 : 0;
  if (len > uint32_t(kTkFastList)) return;  // the whole workgroup
  tk_sort_emit(list, len, kTkFastList, k, tok, out_values, out_indices, rank);
}

template <typename T, bool VEC>
__global__ __launch_bounds__(kTkThreads, 8) void topk_rows_fast_kernel(const T* __restrict__ logits, int64_t stride,
                                                                    int64_t vocab, const int32_t* __restrict__ row_ids,
                                                                    int k, float* __restrict__ out_values,
                                                                    int64_t* __restrict__ out_indices,
                                                                    uint8_t* __restrict__ needs_general) {
  __shared__ uint64_t list[kTkFastList];
  __shared__ uint32_t tot[kTkBins];
  __shared__ uint32_t group_best[kTkGroups];  // largest key of every group of eight consecutive 16-byte vectors
  __shared__ uint32_t rank[kTkRankMax];
  __shared__ uint32_t wave_part[kTkWaves];
  __shared__ uint32_t found[3];
  __shared__ uint32_t count;
  const int tid = threadIdx.x;
  const int64_t tok = blockIdx.x;
  const int64_t row = row_ids ? int64_t(row_ids[tok]) : tok;
  const T* x = logits + row * stride;
  constexpr int VN = Row<T>::kPerVec;
  const int64_t nvec = VEC ? vocab / VN : 0;
  // With 16-byte loads, eight neighbouring lanes read eight neighbouring vectors (128 bytes): the first look also
  // notes each such group's largest key, and the second look skips the groups that lie below the bound -- all but a
  // few per cent of the row.
  const bool by_group = VEC && nvec > 0 && nvec <= int64_t(8) * kTkGroups;

  uint32_t best = 0u;  // below the key of every value
  if (by_group) {
    const u32x4* xv = reinterpret_cast<const u32x4*>(x);
    // A ring of kTkFastBatch vectors in flight: each slot is refilled as soon as its vector has been looked at.
    // Loads past the row's end are clamped to its last vector instead of being skipped (their result is ignored):
    // without a branch around the loads the compiler can count how many may stay in flight at each use.
    const int64_t last = nvec - 1;
    u32x4 raw[kTkFastBatch];
#pragma unroll
    for (int u = 0; u < kTkFastBatch; ++u) {
      const int64_t i = int64_t(tid) + int64_t(u) * kTkThreads;
      raw[u] = xv[i < last ? i : last];
    }
    for (int64_t i0 = tid; i0 - tid < nvec; i0 += int64_t(kTkFastBatch) * kTkThreads) {  // whole waves stay together
      // the ring's loads are awaited here, once per turn (vmcnt(0)): inside the turn every slot is then known to be
      // complete, and the refills issued during it have the rest of the turn to land
      __builtin_amdgcn_s_waitcnt(0x0F70);
#pragma unroll
      for (int u = 0; u < kTkFastBatch; ++u) {
        const int64_t i = i0 + int64_t(u) * kTkThreads;
        // the largest of the vector's values by a float maximum (which passes over NaN) and a NaN flag: one key
        // conversion per vector instead of one per element
        float v[VN];
        Row<T>::unpack(raw[u], v);
        const int64_t ahead = i + int64_t(kTkFastBatch) * kTkThreads;
        raw[u] = xv[ahead < last ? ahead : last];
        float vmax = v[0];
        bool nan = v[0] != v[0];
#pragma unroll
        for (int e = 1; e < VN; ++e) {
          vmax = fmaxf(vmax, v[e]);
          nan |= v[e] != v[e];
        }
        uint32_t top = nan ? 0xFFFFFFFFu : tk_key(vmax);
        top = i < nvec ? top : 0u;
        best = top > best ? top : best;
        {
          uint32_t other = lane_xor<1>(top);
          top = other > top ? other : top;
          other = lane_xor<2>(top);
          top = other > top ? other : top;
          other = lane_xor<4>(top);
          top = other > top ? other : top;
        }
        if ((tid & 7) == 0 && i < nvec) group_best[i >> 3] = top;
      }
    }
    for (int64_t e = nvec * VN + tid; e < vocab; e += kTkThreads) {
      const uint32_t key = tk_key(Row<T>::load1(x + e));
      best = key > best ? key : best;
    }
  } else {
    tk_for_each<T, VEC, false>(x, vocab, [&](uint32_t, float v) {
      const uint32_t key = tk_key(v);
      best = key > best ? key : best;
    });
  }
  uint32_t floor_key;
  const float floor_value = tk_fast_floor(best, k, tot, wave_part, found, &count, &floor_key);
  auto consider = [&](uint32_t idx, float v) { tk_fast_consider(idx, v, floor_value, list, &count); };
  if (by_group) {
    const u32x4* xv = reinterpret_cast<const u32x4*>(x);
    for (int64_t i0 = tid; i0 < nvec; i0 += int64_t(kTkFastBatch) * kTkThreads) {
      u32x4 raw[kTkFastBatch];
      bool wanted[kTkFastBatch];
#pragma unroll
      for (int u = 0; u < kTkFastBatch; ++u) {
        const int64_t i = i0 + int64_t(u) * kTkThreads;
        wanted[u] = i < nvec && group_best[i >> 3] >= floor_key;
        if (wanted[u]) raw[u] = load_stream(xv + i);
      }
#pragma unroll
      for (int u = 0; u < kTkFastBatch; ++u)
        if (wanted[u]) {
          const int64_t i = i0 + int64_t(u) * kTkThreads;
          float v[VN];
          Row<T>::unpack(raw[u], v);
#pragma unroll
          for (int e = 0; e < VN; ++e) consider(uint32_t(i * VN + e), v[e]);
        }
    }
    for (int64_t e = nvec * VN + tid; e < vocab; e += kTkThreads) consider(uint32_t(e), Row<T>::load1(x + e));
  } else {
    tk_for_each<T, VEC, true>(x, vocab, consider);
  }
  tk_fast_finish(list, &count, k, tok, out_values, out_indices, needs_general, rank);
}

// Log-prob + entropy and the top-K ids of a row from ONE read of it (the forward-only pass of an actor that also
// collects its top-K ids, relax/backends/megatron/loss.py:373-446): the softmax scan is scan_row() itself, same
// workgroup width and order as the forward-only kernel, so log-probs and entropy are bit-identical to that kernel's.
// The scan already takes the maximum of every batch of elements a lane absorbs (it rescales its sums by it); its
// observer keeps those maxima, one LDS word per lane and batch, and nothing else is added to the scan.  A lane's
// largest is its thread maximum for the shortcut's bound, and the second look is lane-private: each lane reads again
// only those of its own batches whose maximum reaches the bound (a few per cent of the row, found in the memory-side
// cache).  The bound is taken and those reads are requested right behind the scan, before the workgroup merges its
// softmax state: the round trip then overlaps the merge and thread 0's logarithm (3.53 -> 3.49 ms on 65536 x 151936).  A row that holds NaN or +inf (its sum of exponentials is NaN) goes to the general kernel.
// Built for rows of whole 16-byte vectors whose length selects the 1024-thread scan.
constexpr int kTkScanSlots = 12;  // batches a lane may absorb: vocab / (kScanUnroll * 1024 * elements per vector) + 3

struct TkScanHook {
  float* slot;  // this lane's word of the next batch
  float best;
  __device__ __forceinline__ void absorbed(float vmax) {
    *slot = vmax;
    slot += kTkThreads;
    best = fmaxf(best, vmax);
  }
};

template <typename T>
__global__ __launch_bounds__(kTkThreads, 8) void logprob_topk_fwd_kernel(
    const T* __restrict__ logits, int64_t stride, int64_t vocab, const int32_t* __restrict__ row_ids,
    const int64_t* __restrict__ targets, float c, float inv_t, int k, float* __restrict__ log_prob,
    float* __restrict__ entropy, float* __restrict__ lse_out, float* __restrict__ spx_out,
    float* __restrict__ out_values, int64_t* __restrict__ out_indices, uint8_t* __restrict__ needs_general) {
  __shared__ uint64_t list[kTkFastList];  // the bound's histogram lives here before the candidates do
  __shared__ float lane_max[kTkScanSlots * kTkThreads];
  __shared__ uint32_t rank[kTkRankMax];
  __shared__ uint32_t wave_part[kTkWaves];
  __shared__ uint32_t found[3];
  __shared__ uint32_t count;
  __shared__ uint32_t odd_row;
  __shared__ float wave_state[kTkWaves][3];
  static_assert(sizeof(list) == sizeof(uint32_t) * kTkBins, "the histogram of the thread maxima fits the list");
  uint32_t* tot = reinterpret_cast<uint32_t*>(list);
  const int tid = threadIdx.x;
  const int64_t tok = blockIdx.x;
  const int64_t row = row_ids ? int64_t(row_ids[tok]) : tok;
  const T* x = logits + row * stride;
  constexpr int VN = Row<T>::kPerVec;
  const int64_t nvec = vocab / VN;
  float x_target = 0.f;
  int64_t tg = -1;
  if (tid == 0) {
    tg = targets[tok];
    if (tg >= 0 && tg < vocab) x_target = Row<T>::load1(x + tg);
  }
  TkScanHook hook{lane_max + tid, -__builtin_inff()};
  SoftmaxAcc st = scan_row<T, true, true, kTkThreads>(x, vocab, c, hook);
  uint32_t floor_key;
  const float floor_value = tk_fast_floor(tk_key(hook.best), k, tot, wave_part, found, &count, &floor_key);
  // (tk_fast_floor ends with a barrier after the last reading of tot[]: the list may now overwrite it)
  // Second look, lane-private.  A lane's batches are numbered in the scan's order: `nb` batches of kScanUnroll vectors
  // at a stride of kTkThreads vectors, then single vectors.  Few lanes have a batch that reaches the bound and hardly
  // any has more than two (a few hundred batches qualify in a row of 1024 lanes x 7), so the first two are found from
  // the LDS words alone and their vectors requested together: one memory round trip instead of one per batch.
  const u32x4* xv = reinterpret_cast<const u32x4*>(x);
  const float* mine = lane_max + tid;
  const int nb = nvec >= int64_t(kScanUnroll - 1) * kTkThreads + tid + 1
                     ? int((nvec - int64_t(kScanUnroll - 1) * kTkThreads - tid - 1) / (int64_t(kScanUnroll) * kTkThreads)) + 1
                     : 0;
  const int64_t single0 = int64_t(tid) + int64_t(nb) * kScanUnroll * kTkThreads;  // the lane's first single vector
  const int ns = single0 < nvec ? int((nvec - single0 - 1) / kTkThreads) + 1 : 0;
  auto slot_base = [&](int sl) -> int64_t {
    return sl < nb ? int64_t(tid) + int64_t(sl) * kScanUnroll * kTkThreads : single0 + int64_t(sl - nb) * kTkThreads;
  };
  int hit0 = -1, hit1 = -1, resume = nb + ns;
  for (int sl = 0; sl < nb + ns; ++sl) {
    if (mine[sl * kTkThreads] < floor_value) continue;
    if (hit0 < 0) {
      hit0 = sl;
    } else if (hit1 < 0) {
      hit1 = sl;
    } else {
      resume = sl;
      break;
    }
  }
  auto consider_vec = [&](const u32x4& raw, int64_t i) {
    float v[VN];
    Row<T>::unpack(raw, v);
#pragma unroll
    for (int e = 0; e < VN; ++e) tk_fast_consider(uint32_t(i * VN + e), v[e], floor_value, list, &count);
  };
  u32x4 raw0[kScanUnroll], raw1[kScanUnroll];
  const int64_t b0 = slot_base(hit0 >= 0 ? hit0 : 0), b1 = slot_base(hit1 >= 0 ? hit1 : (hit0 >= 0 ? hit0 : 0));
  const int c0 = hit0 < 0 ? 0 : (hit0 < nb ? kScanUnroll : 1), c1 = hit1 < 0 ? 0 : (hit1 < nb ? kScanUnroll : 1);
  if (hit0 >= 0) {  // a minority of the lanes: their vectors are requested now ...
#pragma unroll
    for (int u = 0; u < kScanUnroll; ++u) {
      if (u < c0) raw0[u] = load_stream(xv + b0 + int64_t(u) * kTkThreads);
      if (u < c1) raw1[u] = load_stream(xv + b1 + int64_t(u) * kTkThreads);
    }
  }
  // ... and travel while the workgroup merges its scan and thread 0 finishes the row's log-prob and entropy
  scan_block_merge<kTkThreads>(st, wave_state);
  if (tid == 0) {
    float lse, spx, ent, lp;
    scan_finish(st, x_target, tg >= 0 && tg < vocab, inv_t, lse, spx, ent, lp);
    log_prob[tok] = lp;
    if (entropy) entropy[tok] = ent;
    if (spx_out) spx_out[tok] = spx;
    if (lse_out) lse_out[tok] = lse;
    odd_row = st.s != st.s ? 1u : 0u;
  }
  __syncthreads();
  if (odd_row) {  // the whole workgroup
    if (tid == 0) needs_general[tok] = 1;
    return;
  }
  if (hit0 >= 0) {
#pragma unroll
    for (int u = 0; u < kScanUnroll; ++u) {
      if (u < c0) consider_vec(raw0[u], b0 + int64_t(u) * kTkThreads);
      if (u < c1) consider_vec(raw1[u], b1 + int64_t(u) * kTkThreads);
    }
    for (int sl = resume; sl < nb + ns; ++sl) {  // a third and further batches of one lane: one at a time
      if (mine[sl * kTkThreads] < floor_value) continue;
      const int64_t b = slot_base(sl);
      const int c = sl < nb ? kScanUnroll : 1;
      for (int u = 0; u < c; ++u) consider_vec(load_stream(xv + b + int64_t(u) * kTkThreads), b + int64_t(u) * kTkThreads);
    }
  }
  tk_fast_finish(list, &count, k, tok, out_values, out_indices, needs_general, rank);
}

// The general way, for the rows the shortcut flagged (long runs of equal or nearly equal values): radix select, 12
// bits at a time.  Persistent workgroups, one per CU, walk the flags.
template <typename T, bool VEC>
__global__ __launch_bounds__(kTkThreads) void topk_rows_kernel(const T* __restrict__ logits, int64_t stride,
                                                               int64_t vocab, const int32_t* __restrict__ row_ids,
                                                               int64_t n_tokens, int k, float* __restrict__ out_values,
                                                               int64_t* __restrict__ out_indices,
                                                               const uint8_t* __restrict__ needs_general) {
  __shared__ uint32_t hist[kTkWaves][kTkBins / 2];  // two 16-bit counters per word; afterwards the (key, index) list
  __shared__ uint32_t tot[kTkBins];
  __shared__ uint32_t wave_part[kTkWaves];
  __shared__ uint32_t found[3];
  __shared__ uint32_t counters[2];  // list length, prefix-sharing keys seen
  __shared__ uint32_t rank[kTkRankMax];
  uint32_t* const hist_words = &hist[0][0];
  uint64_t* const list = reinterpret_cast<uint64_t*>(hist_words);
  const int tid = threadIdx.x, wave = tid / kWave;

  // this workgroup's rows are blockIdx.x, blockIdx.x + gridDim.x, ...; their flags are fetched 1024 at a time, one per
  // thread, so that a launch with nothing to do costs one load instead of a chain of them
  __shared__ uint8_t flagged[kTkThreads];
  for (int64_t chunk = blockIdx.x; chunk < n_tokens; chunk += int64_t(kTkThreads) * gridDim.x) {
    const int64_t mine = chunk + int64_t(tid) * gridDim.x;
    __syncthreads();  // the previous chunk's flags have been walked
    flagged[tid] = mine < n_tokens ? needs_general[mine] : uint8_t(0);
    if (!__syncthreads_or(flagged[tid])) continue;  // nothing flagged among these rows (the usual case)
    for (int slot = 0; slot < kTkThreads; ++slot) {
      if (!flagged[slot]) continue;  // the same answer in every thread
      const int64_t tok = chunk + int64_t(slot) * gridDim.x;
      const int64_t row = row_ids ? int64_t(row_ids[tok]) : tok;
      const T* x = logits + row * stride;
      uint32_t prefix = 0, need = uint32_t(k);
      int prefix_bits = 0;
      while (true) {
        const int db = 32 - prefix_bits < kTkDigitBits ? 32 - prefix_bits : kTkDigitBits;
        for (int i = tid; i < kTkWaves * kTkBins / 2; i += kTkThreads) hist_words[i] = 0u;
        __syncthreads();
        tk_for_each<T, VEC, false>(x, vocab, [&](uint32_t, float v) {
          const uint32_t key = tk_key(v);
          if (prefix_bits == 0 || (key >> (32 - prefix_bits)) == prefix) {
            const uint32_t digit = (key << prefix_bits) >> (32 - db);
            atomicAdd(&hist[wave][digit >> 1], (digit & 1u) ? 0x10000u : 1u);
          }
        });
        __syncthreads();
        for (int d = tid; d < kTkBins; d += kTkThreads) {
          uint32_t sum = 0;
  #pragma unroll
          for (int w = 0; w < kTkWaves; ++w) sum += (hist[w][d >> 1] >> ((d & 1) * 16)) & 0xFFFFu;
          tot[d] = sum;
        }
        __syncthreads();
        tk_locate(tot, wave_part, found, need);
        const uint32_t digit = found[0], above = found[1], inside = found[2];
        prefix = (prefix_bits == 0 ? 0u : prefix << db) | digit;
        prefix_bits += db;
        need -= above;  // how many of the prefix-sharing keys are still wanted: at least one
        if (inside <= uint32_t(kTkCap) || prefix_bits >= 32) break;
      }
      if (tid == 0) counters[0] = counters[1] = 0u;
      __syncthreads();  // also: every thread is done with the histogram, whose memory now holds the list
      tk_for_each<T, VEC, true>(x, vocab, [&](uint32_t idx, float v) {
        const uint32_t key = tk_key(v);
        const uint32_t top = prefix_bits >= 32 ? key : key >> (32 - prefix_bits);
        bool take = top > prefix;
        if (top == prefix) take = atomicAdd(&counters[1], 1u) < uint32_t(kTkCap);
        if (take) {
          const uint32_t slot = atomicAdd(&counters[0], 1u);
          if (slot < uint32_t(kTkList)) list[slot] = (uint64_t(key) << 32) | uint64_t(0xFFFFFFFFu - idx);
        }
      });
      __syncthreads();
      tk_sort_emit(list, counters[0], kTkList, k, tok, out_values, out_indices, rank);
      __syncthreads();  // the list is read to the end before the next row's histogram overwrites it
    }
  }
}

}  // namespace relax_amd

using namespace relax_amd;

template <typename T>
static int launch_topk_rows(const void* logits, int64_t n_tokens, int64_t vocab, int64_t stride,
                            const int32_t* row_ids, int k, float* values, int64_t* indices, uint8_t* flags,
                            hipStream_t s) {
  const bool vec = aligned16(logits) && (stride * int64_t(sizeof(T))) % 16 == 0;
  const T* x = static_cast<const T*>(logits);
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  const dim3 rows(static_cast<unsigned>(n_tokens)), block(kTkThreads);
  const dim3 persistent(static_cast<unsigned>(n_tokens < cus ? n_tokens : cus));
  if (vec) {
    hipLaunchKernelGGL((topk_rows_fast_kernel<T, true>), rows, block, 0, s, x, stride, vocab, row_ids, k, values,
                       indices, flags);
    if (int rc = check_launch("topk_rows_fast")) return rc;
    hipLaunchKernelGGL((topk_rows_kernel<T, true>), persistent, block, 0, s, x, stride, vocab, row_ids, n_tokens, k,
                       values, indices, flags);
  } else {
    hipLaunchKernelGGL((topk_rows_fast_kernel<T, false>), rows, block, 0, s, x, stride, vocab, row_ids, k, values,
                       indices, flags);
    if (int rc = check_launch("topk_rows_fast")) return rc;
    hipLaunchKernelGGL((topk_rows_kernel<T, false>), persistent, block, 0, s, x, stride, vocab, row_ids, n_tokens, k,
                       values, indices, flags);
  }
  return check_launch("topk_rows");
}

extern "C" int relax_amd_topk_rows(const void* logits, int dtype, int64_t n_tokens, int64_t vocab, int64_t row_stride,
                                   const int32_t* row_ids, int k, float* values, int64_t* indices, uint8_t* workspace,
                                   void* stream) {
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (n_tokens < 0 || vocab <= 0 || row_stride < vocab || !logits || !indices || !workspace || k < 1 || k > vocab) {
    set_error("topk_rows: NULL argument, negative size, row_stride < vocab or k outside [1, vocab]");
    return RELAX_AMD_EINVAL;
  }
  if (n_tokens > 0x7FFFFFFFLL) {
    set_error("topk_rows: more than 2^31 - 1 rows in one launch");
    return RELAX_AMD_EINVAL;
  }
  // the wave-private counters are 16 bits wide: a wave sees vocab / 16 elements (+1 vector)
  if (k > kTkMaxK || vocab > 1000000) {
    set_error("topk_rows: k > %d or vocab > 1000000 is not built", kTkMaxK);
    return RELAX_AMD_EUNSUPPORTED;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case RELAX_AMD_F32: return launch_topk_rows<float>(logits, n_tokens, vocab, row_stride, row_ids, k, values, indices, workspace, s);
    case RELAX_AMD_BF16: return launch_topk_rows<bf16_t>(logits, n_tokens, vocab, row_stride, row_ids, k, values, indices, workspace, s);
    case RELAX_AMD_F16: return launch_topk_rows<f16_t>(logits, n_tokens, vocab, row_stride, row_ids, k, values, indices, workspace, s);
    default: set_error("topk_rows: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
}

template <typename T>
static bool topk_fusable(const void* logits, int64_t vocab, int64_t stride) {
  constexpr int per_vec = 16 / int(sizeof(T));
  const int64_t nvec = vocab / per_vec;
  return aligned16(logits) && (stride * int64_t(sizeof(T))) % 16 == 0 && vocab % per_vec == 0 &&
         nvec / (int64_t(kScanUnroll) * kTkThreads) + 3 <= kTkScanSlots && scan_threads(vocab, per_vec) == kTkThreads;
}

template <typename T>
static int launch_logprob_topk(const void* logits, int64_t n_tokens, int64_t vocab, int64_t stride,
                               const int32_t* row_ids, const int64_t* targets, float inv_t, int k, float* log_prob,
                               float* entropy, float* lse, float* spx, float* values, int64_t* indices, uint8_t* flags,
                               hipStream_t s) {
  const T* x = static_cast<const T*>(logits);
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  hipLaunchKernelGGL((logprob_topk_fwd_kernel<T>), dim3(static_cast<unsigned>(n_tokens)), dim3(kTkThreads), 0, s, x,
                     stride, vocab, row_ids, targets, inv_t * kLog2e, inv_t, k, log_prob, entropy, lse, spx, values,
                     indices, flags);
  if (int rc = check_launch("logprob_topk_fwd")) return rc;
  hipLaunchKernelGGL((topk_rows_kernel<T, true>), dim3(static_cast<unsigned>(n_tokens < cus ? n_tokens : cus)),
                     dim3(kTkThreads), 0, s, x, stride, vocab, row_ids, n_tokens, k, values, indices, flags);
  return check_launch("topk_rows");
}

extern "C" int relax_amd_logprob_entropy_topk_fwd(const void* logits, int dtype, int64_t n_tokens, int64_t vocab,
                                                  int64_t row_stride, const int32_t* row_ids, const int64_t* targets,
                                                  float inv_temperature, int k, float* log_prob, float* entropy,
                                                  float* lse, float* spx, float* values, int64_t* indices,
                                                  uint8_t* workspace, void* stream) {
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (n_tokens < 0 || n_tokens > 0x7FFFFFFFLL || vocab <= 0 || row_stride < vocab || !logits || !targets ||
      !log_prob || !indices || !workspace || k < 1 || k > vocab || !(inv_temperature > 0.f)) {
    set_error("logprob_entropy_topk_fwd: NULL argument, bad size, k outside [1, vocab] or non-positive inv_temperature");
    return RELAX_AMD_EINVAL;
  }
  if (k > kTkMaxK || vocab > 1000000) {
    set_error("logprob_entropy_topk_fwd: k > %d or vocab > 1000000 is not built", kTkMaxK);
    return RELAX_AMD_EUNSUPPORTED;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  bool fused = false;
  switch (dtype) {
    case RELAX_AMD_F32: fused = topk_fusable<float>(logits, vocab, row_stride); break;
    case RELAX_AMD_BF16: fused = topk_fusable<bf16_t>(logits, vocab, row_stride); break;
    case RELAX_AMD_F16: fused = topk_fusable<f16_t>(logits, vocab, row_stride); break;
    default: set_error("logprob_entropy_topk_fwd: unknown dtype code %d", dtype); return RELAX_AMD_EINVAL;
  }
  if (!fused) {  // other row shapes: the two passes one after the other, same results
    if (int rc = relax_amd_logprob_entropy_fwd(logits, dtype, n_tokens, vocab, row_stride, row_ids, targets,
                                               inv_temperature, log_prob, entropy, lse, spx, stream))
      return rc;
    return relax_amd_topk_rows(logits, dtype, n_tokens, vocab, row_stride, row_ids, k, values, indices, workspace,
                               stream);
  }
  switch (dtype) {
    case RELAX_AMD_F32:
      return launch_logprob_topk<float>(logits, n_tokens, vocab, row_stride, row_ids, targets, inv_temperature, k,
                                        log_prob, entropy, lse, spx, values, indices, workspace, s);
    case RELAX_AMD_BF16:
      return launch_logprob_topk<bf16_t>(logits, n_tokens, vocab, row_stride, row_ids, targets, inv_temperature, k,
                                         log_prob, entropy, lse, spx, values, indices, workspace, s);
    default:
      return launch_logprob_topk<f16_t>(logits, n_tokens, vocab, row_stride, row_ids, targets, inv_temperature, k,
                                        log_prob, entropy, lse, spx, values, indices, workspace, s);
  }
}
