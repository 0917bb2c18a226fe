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

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
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

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace relax_amd
