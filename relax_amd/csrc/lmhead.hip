// Fused LM-head projection + log-prob / entropy: logits = hidden @ weight^T are produced tile by tile on the bf16
// matrix cores (v_mfma_f32_32x32x16_bf16) and consumed in registers, so the [N, V] logits never reach HBM.
//
// Replaces the deferred-LM-head path of relax/backends/megatron/loss.py:391-419 (per 1024-row sub-chunk:
// F.linear -> .float() -> /T -> calculate_log_probs_and_entropy), and adds the entropy the reference leaves out.
//
// Tiling.  A workgroup (256 threads = 4 wave64) owns 256 tokens and walks a range of 256-wide vocabulary tiles; the
// K loop over the hidden size runs in 32-wide slices, double-buffered through LDS (2 x (256+256) rows x 80 B,
// rows padded by 16 B so the 16-byte fragment reads of 8 consecutive rows hit distinct banks).  The MFMA "A"
// operand is the WEIGHT tile and "B" the HIDDEN tile, so in the 32x32 accumulator layout a lane's column is a TOKEN
// and its 16 registers are 16 vocabulary entries: the online softmax over the vocabulary is then a per-lane
// reduction over 64 accumulator values per token (4 tokens per lane, 12 state registers), with one cross-lane and
// one cross-wave merge at the very end.  Each wave computes 128 vocab x 128 tokens = 4x4 MFMA tiles (256 fp32
// accumulators per lane).  Vocabulary ranges are split over workgroups (flash-decoding style) and merged by a small
// combine kernel; the target logit comes from a gather-dot kernel (one wave per token).
//
// Workgroup -> (XCD, row block, vocab split) mapping: hardware places consecutive workgroup ids round-robin on the
// 8 XCDs; the 32 workgroups resident on one XCD are arranged as (32/S) row blocks x S vocab splits so that hidden
// tiles are shared by S workgroups and weight tiles by 32/S workgroups inside that XCD's L2.
#include "device_utils.h"
#include "relax_amd.h"

namespace relax_amd {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kLmTile = 256;                 // tokens per workgroup == vocab entries per tile
constexpr int kLmBK = 32;                    // hidden-size slice per pipeline stage
constexpr int kLmRow = kLmBK + 8;            // LDS row pitch in bf16: +16 B so 8 consecutive rows hit distinct banks
constexpr int kLmThreads = 256;
constexpr int kLmVecPerRow = kLmBK / 8;                      // 16-byte vectors per slice row
constexpr int kLmRowsPerPass = kLmThreads / kLmVecPerRow;    // rows one pass of the workgroup covers
constexpr int kLmPasses = kLmTile / kLmRowsPerPass;          // 16-byte loads per thread per operand slice
constexpr int kLmStage = 2 * kLmTile * kLmRow;       // bf16 elements per stage (weight rows then hidden rows)
constexpr int kLmLdsBytes = 2 * kLmStage * 2;        // two stages
constexpr int kLmXcds = 8, kLmPerXcd = 32;

struct LmGeom {
  int64_t n_tokens, hidden, vocab, h_stride, w_stride;
  int splits, tiles_per_split, n_tiles, row_blocks;
};

__device__ __forceinline__ bool lm_block_coords(const LmGeom& g, int& rb, int& split) {
  const int id = blockIdx.x;
  const int xcd = id % kLmXcds, slot = (id / kLmXcds) % kLmPerXcd, round = id / (kLmXcds * kLmPerXcd);
  const int rb_per_xcd = kLmPerXcd / g.splits;
  split = slot % g.splits;
  rb = round * (kLmXcds * rb_per_xcd) + xcd * rb_per_xcd + slot / g.splits;
  return rb < g.row_blocks;
}

// Global -> register -> LDS staging of one 256-row x kLmBK-col bf16 slice of an operand.  The tile base is
// wave-uniform; each thread keeps kLmPasses 32-bit element offsets (rows past the ragged edge re-read the last valid
// row; their results are discarded).
struct LmStager {
  const uint16_t* base;
  uint32_t off[kLmPasses];
  u32x4 reg[kLmPasses];
  int lds_off;  // bf16 index of this thread's first row/vec inside an operand tile

  __device__ __forceinline__ void init(const uint16_t* matrix, int64_t stride, int64_t row0, int64_t row_limit) {
    const int r = threadIdx.x / kLmVecPerRow, v = threadIdx.x % kLmVecPerRow;
    base = matrix + row0 * stride;
    const int last = int(row_limit - row0);
#pragma unroll
    for (int i = 0; i < kLmPasses; ++i) {
      const int row = min(r + kLmRowsPerPass * i, last);
      off[i] = uint32_t(row) * uint32_t(stride) + uint32_t(v * 8);
    }
    lds_off = r * kLmRow + v * 8;
  }
  __device__ __forceinline__ void load(int kslice) {
#pragma unroll
    for (int i = 0; i < kLmPasses; ++i)
      reg[i] = *reinterpret_cast<const u32x4*>(base + off[i] + kslice * kLmBK);
  }
  __device__ __forceinline__ void store(uint16_t* tile) const {
#pragma unroll
    for (int i = 0; i < kLmPasses; ++i)
      *reinterpret_cast<u32x4*>(tile + lds_off + i * kLmRowsPerPass * kLmRow) = reg[i];
  }
};

__device__ __forceinline__ void lm_mma_stage(const uint16_t* ws, const uint16_t* hs, int wv, int wt, int lane,
                                             floatx16 (&acc)[4][4]) {
  const int frag = (lane & 31) * kLmRow + (lane >> 5) * 8;
#pragma unroll
  for (int ks = 0; ks < kLmBK / 16; ++ks) {
    bf16x8 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      a[i] = *reinterpret_cast<const bf16x8*>(ws + (wv * 128 + i * 32) * kLmRow + frag + ks * 16);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      b[j] = *reinterpret_cast<const bf16x8*>(hs + (wt * 128 + j * 32) * kLmRow + frag + ks * 16);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
  }
}

// One 256x256 logits tile into `acc` (fp32, un-scaled logits).
__device__ __forceinline__ void lm_tile_gemm(uint16_t* lds, LmStager& wst, LmStager& hst, int nk, int wv, int wt,
                                             int lane, floatx16 (&acc)[4][4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  wst.load(0);
  hst.load(0);
  wst.store(lds);
  hst.store(lds + kLmTile * kLmRow);
  __syncthreads();
  for (int kk = 0; kk < nk; ++kk) {
    uint16_t* cur = lds + (kk & 1) * kLmStage;
    uint16_t* nxt = lds + ((kk + 1) & 1) * kLmStage;
    const bool more = kk + 1 < nk;
    if (more) {
      wst.load(kk + 1);
      hst.load(kk + 1);
    }
    lm_mma_stage(cur, cur + kLmTile * kLmRow, wv, wt, lane, acc);
    if (more) {
      wst.store(nxt);
      hst.store(nxt + kLmTile * kLmRow);
    }
    __syncthreads();
  }
}

// vocabulary index of accumulator register r of MFMA tile i for this lane (relative to the tile's first entry)
__device__ __forceinline__ int lm_vocab_of(int wv, int i, int r, int lane) {
  return wv * 128 + i * 32 + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);
}

// Online-softmax update of one token column with the 16 logits of one 32x32 MFMA tile held by this lane.
// `limit` = number of valid vocabulary entries counted from the tile's first entry (masked variant only).
template <bool MASKED>
__device__ __forceinline__ void lm_absorb_block(const floatx16& blk, int vbase, int limit, float c, float& m, float& s,
                                                float& t) {
  float x[16];
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    x[r] = blk[r];
    if (MASKED && vbase + 8 * (r >> 2) + (r & 3) >= limit) x[r] = kNegHuge;
  }
  float vmax = x[0];
#pragma unroll
  for (int r = 1; r < 16; ++r) vmax = fmaxf(vmax, x[r]);
  const float mc = fmaxf(vmax * c, kNegHuge);
  if (mc > m) {
    const float sc = fast_exp2(m - mc);
    s *= sc;
    t *= sc;
    m = mc;
  }
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const float e = fast_exp2(fmaf(x[r], c, -m));  // masked entries: exp2(-huge) = 0
    s += e;
    t = fmaf(e, (MASKED && x[r] <= kNegHuge) ? 0.f : x[r], t);
  }
}

__global__ __launch_bounds__(kLmThreads, 1) void lmhead_fwd_kernel(const uint16_t* __restrict__ hidden,
                                                                   const uint16_t* __restrict__ weight, LmGeom g,
                                                                   float c, float* __restrict__ partial) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint16_t* lds = reinterpret_cast<uint16_t*>(smem);
  int rb, split;
  if (!lm_block_coords(g, rb, split)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wv = wave >> 1, wt = wave & 1;
  const int64_t tok0 = int64_t(rb) * kLmTile;
  const int nk = int(g.hidden / kLmBK);
  LmStager hst, wst;
  hst.init(hidden, g.h_stride, tok0, g.n_tokens - 1);
  float m[4], s[4], t[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    m[j] = kNegHuge;
    s[j] = 0.f;
    t[j] = 0.f;
  }
  const int vt_begin = split * g.tiles_per_split;
  const int vt_end = min(g.n_tiles, vt_begin + g.tiles_per_split);
  for (int vt = vt_begin; vt < vt_end; ++vt) {
    const int64_t v0 = int64_t(vt) * kLmTile;
    wst.init(weight, g.w_stride, v0, g.vocab - 1);
    floatx16 acc[4][4];
    lm_tile_gemm(lds, wst, hst, nk, wv, wt, lane, acc);
    const int limit = int(min<int64_t>(g.vocab - v0, kLmTile));
    if (limit < kLmTile) {  // ragged last tile: entries past the vocabulary are masked out
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          lm_absorb_block<true>(acc[i][j], wv * 128 + i * 32 + 4 * (lane >> 5), limit, c, m[j], s[j], t[j]);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) lm_absorb_block<false>(acc[i][j], 0, 0, c, m[j], s[j], t[j]);
    }
  }
  // merge the two lane halves (same tokens, different vocab rows), then the two waves sharing the tokens
  float* red = reinterpret_cast<float*>(smem);  // [2 (wv)][256 tokens][3]
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float m2 = __shfl_xor(m[j], 32, kWave), s2 = __shfl_xor(s[j], 32, kWave), t2 = __shfl_xor(t[j], 32, kWave);
    const float mn = fmaxf(m[j], m2);
    const float fa = fast_exp2(m[j] - mn), fb = fast_exp2(m2 - mn);
    s[j] = s[j] * fa + s2 * fb;
    t[j] = t[j] * fa + t2 * fb;
    m[j] = mn;
    if (lane < 32) {
      float* o = red + (wv * kLmTile + wt * 128 + j * 32 + lane) * 3;
      o[0] = m[j];
      o[1] = s[j];
      o[2] = t[j];
    }
  }
  __syncthreads();
  const int64_t tok = tok0 + threadIdx.x;
  if (tok < g.n_tokens) {
    const float* a = red + threadIdx.x * 3;
    const float* b = red + (kLmTile + threadIdx.x) * 3;
    const float mn = fmaxf(a[0], b[0]);
    const float fa = fast_exp2(a[0] - mn), fb = fast_exp2(b[0] - mn);
    float* o = partial + (int64_t(split) * g.n_tokens + tok) * 3;
    o[0] = mn;
    o[1] = a[1] * fa + b[1] * fb;
    o[2] = a[2] * fa + b[2] * fb;
  }
}

// logits[target] per token: one wave per token, fp32 accumulation of bf16 products.
__global__ __launch_bounds__(256) void lmhead_target_logit_kernel(const uint16_t* __restrict__ hidden,
                                                                  const uint16_t* __restrict__ weight, LmGeom g,
                                                                  const int64_t* __restrict__ targets,
                                                                  float* __restrict__ x_target) {
  const int lane = threadIdx.x & 63;
  const int64_t tok = blockIdx.x * 4LL + (threadIdx.x >> 6);
  if (tok >= g.n_tokens) return;
  const int64_t tg = targets[tok];
  if (tg < 0 || tg >= g.vocab) {
    if (lane == 0) x_target[tok] = __builtin_nanf("");
    return;
  }
  const u32x4* h = reinterpret_cast<const u32x4*>(hidden + tok * g.h_stride);
  const u32x4* w = reinterpret_cast<const u32x4*>(weight + tg * g.w_stride);
  float acc = 0.f;
  for (int64_t i = lane; i < g.hidden / 8; i += kWave) {
    float a[8], b[8];
    Row<bf16_t>::unpack(h[i], a);
    Row<bf16_t>::unpack(w[i], b);
#pragma unroll
    for (int k = 0; k < 8; ++k) acc = fmaf(a[k], b[k], acc);
  }
  acc = wave_sum(acc);
  if (lane == 0) x_target[tok] = acc;
}

__global__ __launch_bounds__(256) void lmhead_combine_kernel(const float* __restrict__ partial,
                                                             const float* __restrict__ x_target, int64_t n_tokens,
                                                             int splits, float inv_t, float* __restrict__ log_prob,
                                                             float* __restrict__ entropy, float* __restrict__ lse_out,
                                                             float* __restrict__ spx_out) {
  const int64_t tok = blockIdx.x * 256LL + threadIdx.x;
  if (tok >= n_tokens) return;
  float m = kNegHuge, s = 0.f, t = 0.f;
  for (int k = 0; k < splits; ++k) {
    const float* p = partial + (int64_t(k) * n_tokens + tok) * 3;
    const float mn = fmaxf(m, p[0]);
    const float fa = fast_exp2(m - mn), fb = fast_exp2(p[0] - mn);
    s = s * fa + p[1] * fb;
    t = t * fa + p[2] * fb;
    m = mn;
  }
  const float lse = m * kLn2 + logf(s);
  const float spx = (t / s) * inv_t;
  log_prob[tok] = x_target[tok] * inv_t - lse;
  if (entropy) entropy[tok] = lse - spx;
  if (lse_out) lse_out[tok] = lse;
  if (spx_out) spx_out[tok] = spx;
}

// Backward helper: recompute one [chunk, V] slab of logits on the matrix cores and emit, transposed, the bf16
// gradient w.r.t. the logits  dT[v, n] = inv_T * ( g_lp*(onehot - p) + g_H * p * (spx - x) ),  p = exp(x - lse).
// dT is [vocab, chunk] (token-contiguous) so a lane's 32 neighbours write one 64-byte segment.
__global__ __launch_bounds__(kLmThreads, 1) void lmhead_dlogits_kernel(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ weight, LmGeom g, float c, float inv_t,
    const int64_t* __restrict__ targets, const float* __restrict__ lse, const float* __restrict__ spx,
    const float* __restrict__ g_lp, const float* __restrict__ g_ent, const float* __restrict__ grad_scale_dev,
    uint16_t* __restrict__ d_t, int64_t d_stride) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  uint16_t* lds = reinterpret_cast<uint16_t*>(smem);
  int rb, split;
  if (!lm_block_coords(g, rb, split)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wv = wave >> 1, wt = wave & 1;
  const int64_t tok0 = int64_t(rb) * kLmTile;
  const int nk = int(g.hidden / kLmBK);
  LmStager hst, wst;
  hst.init(hidden, g.h_stride, tok0, g.n_tokens - 1);
  const float gs = grad_scale_dev ? *grad_scale_dev : 1.0f;
  float k0[4], a0[4], a1[4], hot[4];
  int64_t tg[4], tokj[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    tokj[j] = tok0 + wt * 128 + j * 32 + (lane & 31);
    const int64_t tk = tokj[j] < g.n_tokens ? tokj[j] : g.n_tokens - 1;
    const float glp = g_lp[tk] * gs, gh = g_ent ? g_ent[tk] * gs : 0.f;
    const float b = gh * inv_t;
    k0[j] = -lse[tk] * kLog2e;
    a0[j] = -glp * inv_t + (g_ent ? b * spx[tk] : 0.f);
    a1[j] = -b * inv_t;
    hot[j] = glp * inv_t;
    tg[j] = targets[tk];
  }
  const int vt_begin = split * g.tiles_per_split;
  const int vt_end = min(g.n_tiles, vt_begin + g.tiles_per_split);
  for (int vt = vt_begin; vt < vt_end; ++vt) {
    const int64_t v0 = int64_t(vt) * kLmTile;
    wst.init(weight, g.w_stride, v0, g.vocab - 1);
    floatx16 acc[4][4];
    lm_tile_gemm(lds, wst, hst, nk, wv, wt, lane, acc);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (tokj[j] >= g.n_tokens) continue;
        const int64_t vb = v0 + wv * 128 + i * 32 + 4 * (lane >> 5);
        const floatx16 blk = acc[i][j];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t v = vb + 8 * (r >> 2) + (r & 3);
          if (v < g.vocab) {
            const float x = blk[r];
            float d = fast_exp2(fmaf(x, c, k0[j])) * fmaf(x, a1[j], a0[j]);
            if (v == tg[j]) d += hot[j];
            d_t[v * d_stride + tokj[j]] = uint16_t(f32_to_bf16_bits(d));
          }
        }
      }
  }
}

}  // namespace relax_amd

using namespace relax_amd;

static int lm_geometry(const char* what, int dtype, int64_t n, int64_t hidden, int64_t vocab, int64_t h_stride,
                       int64_t w_stride, const void* h, const void* w, LmGeom& g) {
  if (dtype != RELAX_AMD_BF16) {
    set_error("%s: hidden states and weight must be bf16", what);
    return RELAX_AMD_EUNSUPPORTED;
  }
  if (n <= 0 || hidden <= 0 || vocab <= 0 || h_stride < hidden || w_stride < hidden || n > (1LL << 30)) {
    set_error("%s: bad shape n_tokens=%lld hidden=%lld vocab=%lld", what, (long long)n, (long long)hidden,
              (long long)vocab);
    return RELAX_AMD_EINVAL;
  }
  if (hidden % kLmBK != 0 || h_stride % 8 != 0 || w_stride % 8 != 0 || !aligned16(h) || !aligned16(w) ||
      int64_t(kLmTile) * h_stride >= (1LL << 31) || int64_t(kLmTile) * w_stride >= (1LL << 31)) {
    set_error("%s: hidden size must be a multiple of %d and rows 16-byte aligned (hidden=%lld)", what, kLmBK,
              (long long)hidden);
    return RELAX_AMD_EUNSUPPORTED;
  }
  g.n_tokens = n;
  g.hidden = hidden;
  g.vocab = vocab;
  g.h_stride = h_stride;
  g.w_stride = w_stride;
  g.row_blocks = int((n + kLmTile - 1) / kLmTile);
  g.n_tiles = int((vocab + kLmTile - 1) / kLmTile);
  int s = 1;
  while (s < 8 && g.row_blocks * s < 512 && s * 2 <= g.n_tiles) s *= 2;
  g.splits = s;
  g.tiles_per_split = (g.n_tiles + s - 1) / s;
  return RELAX_AMD_OK;
}

static unsigned lm_grid(const LmGeom& g) {
  const int rb_per_round = kLmXcds * (kLmPerXcd / g.splits);
  const int rounds = (g.row_blocks + rb_per_round - 1) / rb_per_round;
  return unsigned(rounds) * kLmXcds * kLmPerXcd;
}

template <typename K>
static int lm_enable_lds(K kernel, const char* what) {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kLmLdsBytes);
  if (e != hipSuccess) {
    set_error("%s: cannot reserve %d bytes of LDS: %s", what, kLmLdsBytes, hipGetErrorString(e));
    return RELAX_AMD_ELAUNCH;
  }
  return RELAX_AMD_OK;
}

extern "C" int64_t relax_amd_lmhead_workspace_bytes(int64_t n_tokens) {
  if (n_tokens <= 0) return 0;
  return (8 * 3 + 1) * n_tokens * int64_t(sizeof(float));
}

extern "C" int relax_amd_lmhead_logprob_fwd(const void* hidden, const void* weight, int dtype, int64_t n_tokens,
                                            int64_t hidden_size, int64_t vocab, int64_t h_stride, int64_t w_stride,
                                            const int64_t* targets, float inv_temperature, void* workspace,
                                            float* log_prob, float* entropy, float* lse, float* spx, void* stream) {
  if (n_tokens == 0) return RELAX_AMD_OK;
  LmGeom g;
  if (int rc = lm_geometry("lmhead_logprob_fwd", dtype, n_tokens, hidden_size, vocab, h_stride, w_stride, hidden,
                           weight, g))
    return rc;
  if (!targets || !workspace || !log_prob || !(inv_temperature > 0.f)) {
    set_error("lmhead_logprob_fwd: NULL argument or non-positive inv_temperature");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* partial = static_cast<float*>(workspace);
  float* x_target = partial + 8 * 3 * n_tokens;
  const uint16_t* h = static_cast<const uint16_t*>(hidden);
  const uint16_t* w = static_cast<const uint16_t*>(weight);
  if (int rc = lm_enable_lds(lmhead_fwd_kernel, "lmhead_logprob_fwd")) return rc;
  hipLaunchKernelGGL(lmhead_target_logit_kernel, dim3(unsigned((n_tokens + 3) / 4)), dim3(256), 0, s, h, w, g, targets,
                     x_target);
  if (int rc = check_launch("lmhead_target_logit")) return rc;
  hipLaunchKernelGGL(lmhead_fwd_kernel, dim3(lm_grid(g)), dim3(kLmThreads), kLmLdsBytes, s, h, w, g,
                     inv_temperature * kLog2e, partial);
  if (int rc = check_launch("lmhead_fwd")) return rc;
  hipLaunchKernelGGL(lmhead_combine_kernel, dim3(unsigned((n_tokens + 255) / 256)), dim3(256), 0, s, partial, x_target,
                     n_tokens, g.splits, inv_temperature, log_prob, entropy, lse, spx);
  return check_launch("lmhead_combine");
}

extern "C" int relax_amd_lmhead_dlogits_t(const void* hidden, const void* weight, int dtype, int64_t n_tokens,
                                          int64_t hidden_size, int64_t vocab, int64_t h_stride, int64_t w_stride,
                                          const int64_t* targets, const float* lse, const float* spx,
                                          const float* g_lp, const float* g_ent, const float* grad_scale_dev,
                                          float inv_temperature, void* d_t, int64_t d_stride, void* stream) {
  if (n_tokens == 0) return RELAX_AMD_OK;
  LmGeom g;
  if (int rc = lm_geometry("lmhead_dlogits_t", dtype, n_tokens, hidden_size, vocab, h_stride, w_stride, hidden,
                           weight, g))
    return rc;
  if (!targets || !lse || !g_lp || !d_t || (g_ent && !spx) || d_stride < n_tokens || !(inv_temperature > 0.f)) {
    set_error("lmhead_dlogits_t: NULL argument, short d_stride or non-positive inv_temperature");
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int rc = lm_enable_lds(lmhead_dlogits_kernel, "lmhead_dlogits_t")) return rc;
  hipLaunchKernelGGL(lmhead_dlogits_kernel, dim3(lm_grid(g)), dim3(kLmThreads), kLmLdsBytes, s,
                     static_cast<const uint16_t*>(hidden), static_cast<const uint16_t*>(weight), g,
                     inv_temperature * kLog2e, inv_temperature, targets, lse, spx, g_lp, g_ent, grad_scale_dev,
                     static_cast<uint16_t*>(d_t), d_stride);
  return check_launch("lmhead_dlogits");
}
