// Device-side helpers shared by the gfx950 kernels: 16-byte vector loads/stores of bf16/f16/f32 rows,
// wave64 shuffles, fixed-order workgroup reductions, and the host-side error plumbing of the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

namespace relax_amd {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kNegHuge = -3.0e38f;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct bf16_t {
  uint16_t bits;
};
struct f16_t {
  _Float16 v;
};

// exp2 / log2 on the hardware transcendental unit (v_exp_f32 / v_log_f32), no range fix-ups.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// round-to-nearest-even fp32 -> bf16 (NaN stays NaN)
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
// two fp32 -> packed bf16 pair with the hardware converter (v_cvt_pk_bf16_f32, round-to-nearest-even)
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const floatx2_t f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

template <typename T>
struct Row;  // traits of a 16-byte vector of T

template <>
struct Row<float> {
  static constexpr int kPerVec = 4;
  __device__ static __forceinline__ void unpack(const u32x4& r, float (&o)[4]) {
    o[0] = __uint_as_float(r.x);
    o[1] = __uint_as_float(r.y);
    o[2] = __uint_as_float(r.z);
    o[3] = __uint_as_float(r.w);
  }
  __device__ static __forceinline__ u32x4 pack(const float (&o)[4]) {
    u32x4 r;
    r.x = __float_as_uint(o[0]);
    r.y = __float_as_uint(o[1]);
    r.z = __float_as_uint(o[2]);
    r.w = __float_as_uint(o[3]);
    return r;
  }
  __device__ static __forceinline__ float load1(const float* p) { return *p; }
  __device__ static __forceinline__ void store1(float* p, float v) { *p = v; }
};

template <>
struct Row<bf16_t> {
  static constexpr int kPerVec = 8;
  __device__ static __forceinline__ void unpack(const u32x4& r, float (&o)[8]) {
    o[0] = bf16_lo(r.x);
    o[1] = bf16_hi(r.x);
    o[2] = bf16_lo(r.y);
    o[3] = bf16_hi(r.y);
    o[4] = bf16_lo(r.z);
    o[5] = bf16_hi(r.z);
    o[6] = bf16_lo(r.w);
    o[7] = bf16_hi(r.w);
  }
  __device__ static __forceinline__ u32x4 pack(const float (&o)[8]) {
    u32x4 r;
    r.x = pack_bf16(o[0], o[1]);
    r.y = pack_bf16(o[2], o[3]);
    r.z = pack_bf16(o[4], o[5]);
    r.w = pack_bf16(o[6], o[7]);
    return r;
  }
  __device__ static __forceinline__ float load1(const bf16_t* p) { return __uint_as_float(uint32_t(p->bits) << 16); }
  __device__ static __forceinline__ void store1(bf16_t* p, float v) { p->bits = uint16_t(f32_to_bf16_bits(v)); }
};

template <>
struct Row<f16_t> {
  static constexpr int kPerVec = 8;
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  __device__ static __forceinline__ void unpack(const u32x4& r, float (&o)[8]) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      h2 h = __builtin_bit_cast(h2, w[i]);
      o[2 * i] = float(h.x);
      o[2 * i + 1] = float(h.y);
    }
  }
  __device__ static __forceinline__ u32x4 pack(const float (&o)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      h2 h;
      h.x = _Float16(o[2 * i]);
      h.y = _Float16(o[2 * i + 1]);
      w[i] = __builtin_bit_cast(uint32_t, h);
    }
    u32x4 r;
    r.x = w[0];
    r.y = w[1];
    r.z = w[2];
    r.w = w[3];
    return r;
  }
  __device__ static __forceinline__ float load1(const f16_t* p) { return float(p->v); }
  __device__ static __forceinline__ void store1(f16_t* p, float v) { p->v = _Float16(v); }
};

// streaming (non-temporal) 16-byte accesses: every logits row is touched once per pass
__device__ __forceinline__ u32x4 load_stream(const u32x4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void store_stream(u32x4* p, const u32x4& v) { __builtin_nontemporal_store(v, p); }

// Value that lane (this lane ^ O) of the wave holds, O a power of two below 64: the exchange of __shfl_xor() done by
// cross-lane moves inside the vector ALU (quad permutes, row rotates / mirrors, the 16- and 32-lane swaps) instead
// of a trip through the LDS crossbar, which a wave with nothing else to do waits some hundred cycles for, six times
// per reduction.  Every lane of the wave must be active.
typedef unsigned lane_pair_t __attribute__((ext_vector_type(2)));
template <int O>
__device__ __forceinline__ uint32_t lane_xor(uint32_t b) {
  static_assert(O == 32 || O == 16 || O == 8 || O == 4 || O == 2 || O == 1, "one bit of the lane index");
  if constexpr (O == 32) {
    // both halves of the wave in both results: r[0] = (low, low), r[1] = (high, high)
    const lane_pair_t r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
    return (threadIdx.x & 32) ? r[0] : r[1];
  } else if constexpr (O == 16) {
    // rows of 16 lanes: r[0] = (row 0, row 0, row 2, row 2), r[1] = (row 1, row 1, row 3, row 3)
    const lane_pair_t r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
    return (threadIdx.x & 16) ? r[0] : r[1];
  } else if constexpr (O == 8) {
    return uint32_t(__builtin_amdgcn_update_dpp(0, int(b), 0x128, 0xF, 0xF, true));  // row_ror:8
  } else if constexpr (O == 4) {
    const int h = __builtin_amdgcn_update_dpp(0, int(b), 0x141, 0xF, 0xF, true);  // row_half_mirror: i -> 7 - i
    return uint32_t(__builtin_amdgcn_update_dpp(0, h, 0x1B, 0xF, 0xF, true));      // quad_perm [3, 2, 1, 0]
  } else if constexpr (O == 2) {
    return uint32_t(__builtin_amdgcn_update_dpp(0, int(b), 0x4E, 0xF, 0xF, true));  // quad_perm [2, 3, 0, 1]
  } else {
    return uint32_t(__builtin_amdgcn_update_dpp(0, int(b), 0xB1, 0xF, 0xF, true));  // quad_perm [1, 0, 3, 2]
  }
}
template <int O>
__device__ __forceinline__ float lane_xor(float v) {
  return __uint_as_float(lane_xor<O>(__float_as_uint(v)));
}
template <int O>
__device__ __forceinline__ uint64_t lane_xor(uint64_t v) {
  return uint64_t(lane_xor<O>(uint32_t(v))) | (uint64_t(lane_xor<O>(uint32_t(v >> 32))) << 32);
}
template <int O>
__device__ __forceinline__ double lane_xor(double v) {
  return __longlong_as_double((long long)lane_xor<O>(uint64_t(__double_as_longlong(v))));
}
template <int O>
__device__ __forceinline__ long long lane_xor(long long v) {
  return (long long)lane_xor<O>(uint64_t(v));
}

// The wave64 xor butterfly: step(lane distance as an integral constant) for 32, 16, 8, 4, 2, 1 in this order.
template <int O>
struct LaneDistance {
  static constexpr int value = O;
};
template <typename Step>
__device__ __forceinline__ void wave_butterfly(Step&& step) {
  step(LaneDistance<32>{});
  step(LaneDistance<16>{});
  step(LaneDistance<8>{});
  step(LaneDistance<4>{});
  step(LaneDistance<2>{});
  step(LaneDistance<1>{});
}

// lane `LANE`'s value in every lane
template <int LANE = 0>
__device__ __forceinline__ float lane_value(float v) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), LANE));
}

__device__ __forceinline__ float wave_sum(float v) {
  wave_butterfly([&](auto o) { v += lane_xor<decltype(o)::value>(v); });
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
  wave_butterfly([&](auto o) { v += lane_xor<decltype(o)::value>(v); });
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  wave_butterfly([&](auto o) { v = fmaxf(v, lane_xor<decltype(o)::value>(v)); });
  return v;
}

// Workgroup sum with a fixed combination order (deterministic); result valid in every thread.
// `scratch` holds one slot per wave; THREADS must be a multiple of 64.
template <int THREADS, typename F>
__device__ __forceinline__ F block_sum(F v, F* scratch) {
  constexpr int kWaves = THREADS / kWave;
  v = wave_sum(v);
  const int lane = threadIdx.x & (kWave - 1), w = threadIdx.x / kWave;
  __syncthreads();  // scratch may still be read from a previous call
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  F total = scratch[0];
#pragma unroll
  for (int i = 1; i < kWaves; ++i) total += scratch[i];
  return total;
}

// ---- host side ------------------------------------------------------------------------------------------------
void set_error(const char* fmt, ...);
int check_launch(const char* what);
// RELAX_AMD_KERNEL_* as last set through relax_amd_set_kernel_choice (one relaxed atomic load)
int kernel_choice();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace relax_amd
