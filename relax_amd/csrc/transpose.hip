// out[c, r] = in[r, c] for 16-bit elements: the layout change `x.t().contiguous()` makes, at HBM speed.
//
// The LM-head backward hands the library GEMMs operands whose contraction index is the contiguous one (they run
// 10 - 15 % faster that way); that needs a transposed copy of the [vocab, hidden] weight per backward pass, which the
// framework's generic strided copy does at a few hundred GB/s.  Here a workgroup moves one 64 x 64 tile through LDS:
// 16-byte reads along the input rows, 16-byte writes along the output rows.
#include "device_utils.h"
#include "relax_amd.h"

namespace relax_amd {

constexpr int kTrTile = 64;
constexpr int kTrThreads = 256;
// one extra 32-bit word per LDS row: the eight lanes that gather one output vector walk rows 8 apart and land in banks
// 8 apart; neighbouring output rows share a word (a broadcast), so the gather is conflict-free
constexpr int kTrPitch = kTrTile + 2;

template <bool VEC_IN, bool VEC_OUT>
__global__ __launch_bounds__(kTrThreads) void transpose16_kernel(const uint16_t* __restrict__ in, int64_t rows,
                                                                 int64_t cols, int64_t in_stride,
                                                                 uint16_t* __restrict__ out, int64_t out_stride,
                                                                 int64_t col_tiles) {
  __shared__ __attribute__((aligned(16))) uint16_t tile[kTrTile][kTrPitch];
  const int64_t r0 = (blockIdx.x / col_tiles) * kTrTile, c0 = (blockIdx.x % col_tiles) * kTrTile;
  const int sub = threadIdx.x >> 3, vec = (threadIdx.x & 7) * 8;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int row = sub + 32 * pass;
    const int64_t r = r0 + row, c = c0 + vec;
    uint32_t* dst = reinterpret_cast<uint32_t*>(&tile[row][vec]);  // (row * 66 + vec) * 2 bytes: 4-byte aligned
    if (VEC_IN && r < rows && c + 8 <= cols) {
      const u32x4 v = *reinterpret_cast<const u32x4*>(in + r * in_stride + c);
      dst[0] = v.x, dst[1] = v.y, dst[2] = v.z, dst[3] = v.w;
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k) tile[row][vec + k] = (r < rows && c + k < cols) ? in[r * in_stride + c + k] : 0;
    }
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int ocol = sub + 32 * pass;  // input column = output row
    const int64_t c = c0 + ocol, r = r0 + vec;
    if (c >= cols || r >= rows) continue;
    uint16_t e[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) e[k] = tile[vec + k][ocol];
    if (VEC_OUT && r + 8 <= rows) {
      u32x4 v;
      v.x = e[0] | (uint32_t(e[1]) << 16), v.y = e[2] | (uint32_t(e[3]) << 16);
      v.z = e[4] | (uint32_t(e[5]) << 16), v.w = e[6] | (uint32_t(e[7]) << 16);
      *reinterpret_cast<u32x4*>(out + c * out_stride + r) = v;
    } else {
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (r + k < rows) out[c * out_stride + r + k] = e[k];
    }
  }
}

}  // namespace relax_amd

using namespace relax_amd;

extern "C" int relax_amd_transpose_16bit(const void* in, int64_t rows, int64_t cols, int64_t in_stride, void* out,
                                         int64_t out_stride, void* stream) {
  if (rows == 0 || cols == 0) return RELAX_AMD_OK;
  if (rows < 0 || cols < 0 || !in || !out || in_stride < cols || out_stride < rows) {
    set_error("transpose_16bit: bad arguments rows=%lld cols=%lld in_stride=%lld out_stride=%lld", (long long)rows,
              (long long)cols, (long long)in_stride, (long long)out_stride);
    return RELAX_AMD_EINVAL;
  }
  const int64_t row_tiles = (rows + kTrTile - 1) / kTrTile, col_tiles = (cols + kTrTile - 1) / kTrTile;
  if (row_tiles * col_tiles > 2147483647LL) {
    set_error("transpose_16bit: matrix too large (%lld x %lld)", (long long)rows, (long long)cols);
    return RELAX_AMD_EUNSUPPORTED;
  }
  const bool vin = in_stride % 8 == 0 && aligned16(in), vout = out_stride % 8 == 0 && aligned16(out);
  const dim3 grid(unsigned(row_tiles * col_tiles)), block(kTrThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint16_t* i = static_cast<const uint16_t*>(in);
  uint16_t* o = static_cast<uint16_t*>(out);
  if (vin && vout)
    hipLaunchKernelGGL((transpose16_kernel<true, true>), grid, block, 0, s, i, rows, cols, in_stride, o, out_stride,
                       col_tiles);
  else if (vin)
    hipLaunchKernelGGL((transpose16_kernel<true, false>), grid, block, 0, s, i, rows, cols, in_stride, o, out_stride,
                       col_tiles);
  else if (vout)
    hipLaunchKernelGGL((transpose16_kernel<false, true>), grid, block, 0, s, i, rows, cols, in_stride, o, out_stride,
                       col_tiles);
  else
    hipLaunchKernelGGL((transpose16_kernel<false, false>), grid, block, 0, s, i, rows, cols, in_stride, o, out_stride,
                       col_tiles);
  return check_launch("transpose_16bit");
}
