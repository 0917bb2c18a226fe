// Measurement aids, not part of the loss path and not part of the product library: built into their own small
// library (libceilings.so), which only the benchmark loads.  Entry points return 0, -1 for bad arguments, or the HIP
// error code of a failed launch.
//
// (1) The matrix cores fed from registers, with no memory traffic at all.
//
// The published bf16 peak assumes the 2.4 GHz boost clock.  On dense operands with the statistics of real activations
// the board reaches its power limit long before that, so the number a GEMM-shaped kernel can be held against on a
// given box is what this loop sustains there: 64 independent 32x32x16 bf16 MFMAs per iteration and wave, one wave per
// SIMD, operand fragments loaded once from `src` and rotated between the MFMAs so that consecutive instructions see
// different operands, as they do in the LM-head kernels.
#include "device_utils.h"

namespace relax_amd {

typedef __bf16 diag_bf16x8 __attribute__((ext_vector_type(8)));
typedef float diag_floatx16 __attribute__((ext_vector_type(16)));

__global__ __launch_bounds__(256, 1) void diag_mfma_loop_kernel(const diag_bf16x8* __restrict__ src,
                                                                float* __restrict__ out, int iters) {
  const int lane = threadIdx.x;
  diag_bf16x8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = src[i * 256 + lane];
    b[i] = src[(i + 8) * 256 + lane];
  }
  diag_floatx16 acc[4][4] = {};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] =
              __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(i + ks) & 7], b[(j + 2 * ks) & 7], acc[i][j], 0, 0, 0);
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
  out[blockIdx.x * 256 + lane] = sum;
}

// The same measurement for the 16x16x32 shape.  One wave per SIMD cannot issue these four-pass instructions back to
// back (measured 66 % of the issue slots), so this variant runs two waves per SIMD with 32 four-register accumulators
// each: 128 MFMAs of 16x16x32 per iteration and wave, i.e. the same FLOP per iteration as the 32x32x16 loop.
typedef float diag_floatx4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(512, 1) void diag_mfma_loop16_kernel(const diag_bf16x8* __restrict__ src,
                                                                  float* __restrict__ out, int iters) {
  const int lane = threadIdx.x & 255;
  diag_bf16x8 a[8], b[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = src[i * 256 + lane];
    b[i] = src[(i + 8) * 256 + lane];
  }
  diag_floatx4 acc[4][8] = {};
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j)
          acc[i][j] =
              __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[(i + ks) & 7], b[(j + 3 * ks) & 7], acc[i][j], 0, 0, 0);
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j)
#pragma unroll
      for (int r = 0; r < 4; ++r) sum += acc[i][j][r];
  out[blockIdx.x * 512 + threadIdx.x] = sum;
}

// Plain HBM streams, for the ceiling the bandwidth-bound kernels can be held against on a given box: 16-byte accesses,
// four in flight per thread, grid-stride over the buffer.  mode 0 reads, 1 writes, 2 copies.
template <int MODE>
__global__ __launch_bounds__(1024) void diag_stream_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out,
                                                           int64_t n, unsigned* __restrict__ sink) {
  constexpr int kUnroll = 4;
  int64_t i = int64_t(blockIdx.x) * 1024 * kUnroll + threadIdx.x;
  const int64_t stride = int64_t(gridDim.x) * 1024 * kUnroll;
  unsigned acc = 0;
  for (; i + 1024 * (kUnroll - 1) < n; i += stride) {
    u32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (MODE == 1)
        v[u] = u32x4{unsigned(i), 2u, 3u, 4u};
      else
        v[u] = __builtin_nontemporal_load(in + i + u * 1024);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (MODE == 0)
        acc += v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
      else
        __builtin_nontemporal_store(v[u], out + i + u * 1024);
    }
  }
  if (MODE == 0 && acc == 0x12345678u) sink[0] = acc;  // keeps the loads alive; practically never true
}

// Write stream in its fastest measured form: 256-thread workgroups that write 4 KB each and exit (6.85 TB/s against
// 5.8 - 6.0 TB/s for any form in which a workgroup writes 16 KB or more: the more compact the window of addresses
// being written at one time, the higher the rate).
__global__ __launch_bounds__(256) void diag_write_oneshot_kernel(u32x4* __restrict__ out) {
  const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
  out[i] = u32x4{unsigned(i), 2u, 3u, 4u};
}

// The same copy walked the way the row kernels walk memory: rows of `row_vecs` 16-byte vectors, workgroup b takes
// rows b, b + gridDim, ... and streams each row from end to end.  Compared with the grid-stride copy above it shows
// what the one-workgroup-per-row access pattern itself costs on a given box.
__global__ __launch_bounds__(1024) void diag_row_copy_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out,
                                                             int64_t rows, int64_t row_vecs) {
  for (int64_t r = blockIdx.x; r < rows; r += gridDim.x) {
    const u32x4* ip = in + r * row_vecs;
    u32x4* op = out + r * row_vecs;
    for (int64_t i = threadIdx.x; i < row_vecs; i += 1024)
      __builtin_nontemporal_store(__builtin_nontemporal_load(ip + i), op + i);
  }
}

// The copy in the burst form of the register-resident kernels: persistent workgroups, a whole row into the registers
// by one run of loads, out again by one run of stores, the next row's loads issued right behind them.  Nothing else:
// what this sustains is the ceiling of those kernels' memory pattern.  THREADS x NV vectors hold a row (rows shorter
// than that leave the last positions partly empty), OCC workgroups share a CU.  With ALIGN the workgroups of the
// whole grid keep in step: each announces that its loads are issued and waits, for a bounded number of polls, until
// all have done so before its stores go out (phases[0] counts the announcements, phases[1] is set when a wait ran
// out, after which nobody waits any more, phases[2] counts such waits).
template <int THREADS, int NV, int OCC, bool ALIGN>
__global__ __launch_bounds__(THREADS, OCC) void diag_burst_copy_kernel(const u32x4* __restrict__ in,
                                                                       u32x4* __restrict__ out, int64_t rows,
                                                                       int64_t row_vecs, unsigned* phases) {
  const int tid = threadIdx.x;
  u32x4 reg[NV];
  int64_t row = blockIdx.x;
  if (row >= rows) return;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int64_t v = tid + j * THREADS;
    reg[j] = __builtin_nontemporal_load(in + row * row_vecs + (v < row_vecs ? v : 0));
  }
  unsigned turn = 0;
  if (ALIGN && tid == 0) __hip_atomic_fetch_add(&phases[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (true) {
    __syncthreads();  // as the row kernels: the row is complete in the registers behind their barrier
    if (ALIGN) {
      if (tid == 0 && !__hip_atomic_load(&phases[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
        const unsigned target = (turn + 1) * gridDim.x;
        int polls = 0;
        while (__hip_atomic_load(&phases[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
          if (++polls > 3000) {  // a few milliseconds: workgroups that are not co-resident, or an uneven row count
            __hip_atomic_store(&phases[1], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_fetch_add(&phases[2], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            break;
          }
          __builtin_amdgcn_s_sleep(4);
        }
      }
      __syncthreads();
    }
    const int64_t next = row + gridDim.x;
    const bool has_next = next < rows;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int64_t v = tid + j * THREADS;
      if (v < row_vecs) __builtin_nontemporal_store(reg[j], out + row * row_vecs + v);
    }
    const int64_t src = has_next ? next : row;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int64_t v = tid + j * THREADS;
      reg[j] = __builtin_nontemporal_load(in + src * row_vecs + (v < row_vecs ? v : 0));
    }
    ++turn;
    if (ALIGN && tid == 0) __hip_atomic_fetch_add(&phases[0], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (!has_next) return;
    row = next;
  }
}

}  // namespace relax_amd

using namespace relax_amd;

// mode 3 of the stream probe: row-wise copy with `blocks` persistent workgroups
extern "C" int ceiling_row_copy(const void* src, void* dst, int64_t rows, int64_t row_bytes, int blocks, void* stream) {
  if (!src || !dst || rows < 0 || row_bytes <= 0 || row_bytes % 16 != 0 || blocks <= 0 || !aligned16(src) ||
      !aligned16(dst))
    return -1;
  if (rows == 0) return 0;
  hipLaunchKernelGGL(diag_row_copy_kernel, dim3(unsigned(blocks)), dim3(1024), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4*>(src), static_cast<u32x4*>(dst), rows, row_bytes / 16);
  return int(hipGetLastError());
}

extern "C" int ceiling_stream(int mode, const void* src, void* dst, int64_t bytes, void* sink, void* stream) {
  if (mode < 0 || mode > 2 || bytes < 0 || bytes % (16 * 4096) != 0 || (mode != 1 && !src) || (mode != 0 && !dst) ||
      (mode == 0 && !sink) || !aligned16(src) || !aligned16(dst)) {
    return -1;
  }
  if (bytes == 0) return 0;
  const int64_t n = bytes / 16;
  const int64_t groups = n / 4096;
  const dim3 grid(unsigned(groups < 65536 ? groups : 65536)), block(1024);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const u32x4* in = static_cast<const u32x4*>(src);
  u32x4* out = static_cast<u32x4*>(dst);
  if (mode == 0)
    hipLaunchKernelGGL(diag_stream_kernel<0>, grid, block, 0, s, in, out, n, static_cast<unsigned*>(sink));
  else if (mode == 1 && n / 256 <= 2147483647LL)
    hipLaunchKernelGGL(diag_write_oneshot_kernel, dim3(unsigned(n / 256)), dim3(256), 0, s, out);
  else if (mode == 1)
    hipLaunchKernelGGL(diag_stream_kernel<1>, grid, block, 0, s, in, out, n, static_cast<unsigned*>(sink));
  else
    hipLaunchKernelGGL(diag_stream_kernel<2>, grid, block, 0, s, in, out, n, static_cast<unsigned*>(sink));
  return int(hipGetLastError());
}

extern "C" int ceiling_mfma_loop(const void* src, float* out, int blocks, int iters, int shape, void* stream) {
  if (!src || !out || blocks <= 0 || iters < 0 || !aligned16(src) || (shape != 0 && shape != 1)) {
    return -1;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (shape == 0)
    hipLaunchKernelGGL(diag_mfma_loop_kernel, dim3(unsigned(blocks)), dim3(256), 0, s,
                       static_cast<const diag_bf16x8*>(src), out, iters);
  else
    hipLaunchKernelGGL(diag_mfma_loop16_kernel, dim3(unsigned(blocks)), dim3(512), 0, s,
                       static_cast<const diag_bf16x8*>(src), out, iters);
  return int(hipGetLastError());
}

// Burst-form copy of `rows` rows of `row_bytes` bytes.  threads = 1024 or 512 per workgroup, per_cu = 1 or 2
// persistent workgroups per CU; rows of up to 8 (1024 threads) / 16 (512 threads) vectors per thread take the short
// shape, longer ones (1024 threads only) 19 vectors per thread.  align != 0: the phase-aligned form, `phases` = three
// zeroed 32-bit words of device memory (see the kernel).
extern "C" int ceiling_burst_copy(const void* src, void* dst, int64_t rows, int64_t row_bytes, int threads, int per_cu,
                                  int align, unsigned* phases, void* stream) {
  if (!src || !dst || rows < 0 || row_bytes <= 0 || row_bytes % 16 != 0 || !aligned16(src) || !aligned16(dst) ||
      (threads != 1024 && threads != 512) || (per_cu != 1 && per_cu != 2) || (align && !phases))
    return -1;
  if (rows == 0) return 0;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    return -1;
  const int64_t row_vecs = row_bytes / 16;
  const int64_t slots = int64_t(cus) * per_cu;
  const dim3 grid(unsigned(rows < slots ? rows : slots));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const u32x4* in = static_cast<const u32x4*>(src);
  u32x4* out = static_cast<u32x4*>(dst);
#define RELAX_AMD_BURST(THREADS, NV, OCC)                                                                          \
  if (threads == THREADS && per_cu == OCC && row_vecs <= int64_t(THREADS) * NV) {                                   \
    if (align)                                                                                                      \
      hipLaunchKernelGGL((diag_burst_copy_kernel<THREADS, NV, OCC, true>), grid, dim3(THREADS), 0, s, in, out, rows, \
                         row_vecs, phases);                                                                         \
    else                                                                                                            \
      hipLaunchKernelGGL((diag_burst_copy_kernel<THREADS, NV, OCC, false>), grid, dim3(THREADS), 0, s, in, out,      \
                         rows, row_vecs, phases);                                                                   \
    return int(hipGetLastError());                                                                                  \
  }
  RELAX_AMD_BURST(1024, 8, 1)
  RELAX_AMD_BURST(1024, 8, 2)
  RELAX_AMD_BURST(512, 16, 2)
  RELAX_AMD_BURST(512, 16, 1)
  RELAX_AMD_BURST(1024, 19, 1)
#undef RELAX_AMD_BURST
  return -1;
}
