// Measurement aid, not part of the loss path: the matrix cores fed from registers, with no memory traffic at all.
//
// The published bf16 peak assumes the 2.4 GHz boost clock.  On dense operands with the statistics of real activations
// the board reaches its power limit long before that, so the number a GEMM-shaped kernel can be held against on a
// given box is what this loop sustains there: 64 independent 32x32x16 bf16 MFMAs per iteration and wave, one wave per
// SIMD, operand fragments loaded once from `src` and rotated between the MFMAs so that consecutive instructions see
// different operands, as they do in the LM-head kernels.
#include "device_utils.h"
#include "relax_amd.h"

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

}  // namespace relax_amd

using namespace relax_amd;

extern "C" int relax_amd_diag_mfma_loop(const void* src, float* out, int blocks, int iters, int shape, void* stream) {
  if (!src || !out || blocks <= 0 || iters < 0 || !aligned16(src) || (shape != 0 && shape != 1)) {
    set_error("diag_mfma_loop: src (4096 x 16 bytes, 16-byte aligned), out (blocks x 512 floats) and shape 0 "
              "(32x32x16, one wave per SIMD) or 1 (16x16x32, two waves per SIMD) are required");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (shape == 0)
    hipLaunchKernelGGL(diag_mfma_loop_kernel, dim3(unsigned(blocks)), dim3(256), 0, s,
                       static_cast<const diag_bf16x8*>(src), out, iters);
  else
    hipLaunchKernelGGL(diag_mfma_loop16_kernel, dim3(unsigned(blocks)), dim3(512), 0, s,
                       static_cast<const diag_bf16x8*>(src), out, iters);
  return check_launch("diag_mfma_loop");
}
