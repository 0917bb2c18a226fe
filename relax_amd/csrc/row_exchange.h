// Exchange of per-wave partial results between the one-shot workgroups that share a row (actor_step_split.hip,
// reverse_kl_split.hip).
//
// A ring of slots in device memory, one per (row mod kRing); a slot holds, for each of the row's waves, a few eight-byte
// words, each a float and a 32-bit tag, written and read with relaxed device-scope atomics.  The tag names the launch and
// the lap of the ring: it is derived from a device word behind the ring that a one-workgroup kernel in front of every
// launch advances (so a captured launch gets fresh tags on every replay), and a reader tells a stale word from the one
// it waits for without any fence.  The workgroups of a row have consecutive indices; a workgroup only waits for
// those, which are resident or next in dispatch order whatever else the chip runs, so every wait ends.  It is bounded
// all the same: the first wait of a launch that gives up raises a flag that ends the launch's other waits at their
// next look at it, and counts itself.  A ring is one array per kernel family, process and GPU: launches of one family
// that overlap on one GPU (two streams of one process) can overwrite each other's slots or tags, which ends as such a
// give-up, never as a wrong number taken for right.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <mutex>

#include "device_utils.h"
#include "relax_amd.h"

namespace relax_amd {

constexpr unsigned kRing = 4096;           // rows whose slots exist at a time
constexpr unsigned kWaitPolls = 1u << 17;  // looks at a neighbour's word before a wait gives up (a few suffice; each takes microseconds)
// behind a ring's slots: 32-bit words [0] the tag counter, [1] the count of waits that gave up, [2] the flag the
// first give-up of a launch raises
constexpr int kRingTailWords = 32;

// relax_amd_set_exchange_wait(): the bound of a wait and an offset added to the tag it waits for
unsigned exchange_max_polls();
unsigned exchange_wait_tag_offset();

// Advances the tag counter by the laps of the launch that follows; clears the ring when the 32-bit counter would wrap
// (a tag of a past lap could otherwise come round again), and with it `extra` (a second array of tagged words that
// shares the ring's tags, or null).
template <size_t RING_WORDS>
__global__ __launch_bounds__(256) void exchange_ring_advance_kernel(unsigned long long* ring, unsigned laps,
                                                                    unsigned long long* extra, size_t extra_words) {
  unsigned* counter = reinterpret_cast<unsigned*>(ring + RING_WORDS);
  const unsigned now = counter[0];
  const bool wrap = now > 0xffffffffu - laps - 1u;
  if (wrap) {
    for (size_t i = threadIdx.x; i < RING_WORDS; i += 256) ring[i] = 0ull;
    if (extra)
      for (size_t i = threadIdx.x; i < extra_words; i += 256) extra[i] = 0ull;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    counter[0] = (wrap ? 0u : now) + laps;
    counter[2] = 0u;  // no wait of the launch that follows has given up yet
  }
}

// this launch's tag for `row`: the counter was advanced by `laps` in front of the launch
__device__ __forceinline__ unsigned exchange_tag(const unsigned* status, unsigned laps, int64_t row) {
  return status[0] - laps + 1u + unsigned(row / kRing);
}

__device__ __forceinline__ void exchange_store(unsigned long long* word, unsigned tag, float val) {
  __hip_atomic_store(word, (static_cast<unsigned long long>(tag) << 32) | __float_as_uint(val), __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_AGENT);
}

// Waits, boundedly, for `word` to carry `tag`; false when the wait gave up (its own bound, or another wait's flag).
__device__ __forceinline__ bool exchange_wait(const unsigned long long* word, unsigned tag, unsigned max_polls,
                                              unsigned* status, float& out) {
  unsigned polls = 0;
  while (true) {
    const unsigned long long w = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (unsigned(w >> 32) == tag) {
      out = __uint_as_float(unsigned(w));
      return true;
    }
    ++polls;
    if (polls > max_polls ||
        ((polls & 63u) == 0u && __hip_atomic_load(status + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u))
      return false;
    __builtin_amdgcn_s_sleep(1);
  }
}

// one lane of a wave whose wait gave up: counts it and ends the launch's other waits
__device__ __forceinline__ void exchange_report_give_up(unsigned* status) {
  atomicAdd(status + 1, 1u);
  __hip_atomic_store(status + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The current device's copy of a ring (a file-scope __device__ array): looked up once per device, with that device
// current.
struct ExchangeRingCache {
  static constexpr int kMaxDevices = 64;
  std::mutex mutex;
  unsigned long long* ptr[kMaxDevices] = {};
};
inline int exchange_ring_of_device(ExchangeRingCache& cache, const void* symbol, const char* who,
                                   unsigned long long** ring) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= ExchangeRingCache::kMaxDevices) {
    set_error("%s: no usable current device (%s)", who, e == hipSuccess ? "index out of range" : hipGetErrorString(e));
    return RELAX_AMD_EINVAL;
  }
  std::lock_guard<std::mutex> lock(cache.mutex);
  if (!cache.ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, symbol);
    if (e != hipSuccess || !p) {
      set_error("%s: hipGetSymbolAddress failed on device %d: %s", who, dev, hipGetErrorString(e));
      return RELAX_AMD_ELAUNCH;
    }
    cache.ptr[dev] = static_cast<unsigned long long*>(p);
  }
  *ring = cache.ptr[dev];
  return RELAX_AMD_OK;
}

}  // namespace relax_amd
