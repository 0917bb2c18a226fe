// Fused LM-head projection + log-prob / entropy: logits = hidden @ weight^T are produced tile by tile on the bf16
// matrix cores (v_mfma_f32_32x32x16_bf16) and consumed in registers, so the [N, V] logits never reach HBM.
//
// Replaces the deferred-LM-head path of relax/backends/megatron/loss.py:391-419 (per 1024-row sub-chunk:
// F.linear -> .float() -> /T -> calculate_log_probs_and_entropy), and adds the entropy the reference leaves out.
//
// Tiling.  A workgroup (256 threads = 4 wave64) owns 256 tokens and walks a range of 256-wide vocabulary tiles; the
// K loop over the hidden size runs in 64-wide slices through a two-stage LDS ring (2 x (256 + 256) rows x 128 B).
// Slices are copied global -> LDS directly (global_load_lds_dwordx4, no staging registers): every lane fetches one
// 16-byte vector and the wave's 64 vectors land contiguously, i.e. 8 rows x 128 B per instruction.  The LDS has 64
// four-byte banks and serves 16 lanes of a 16-byte read per clock, so the fragment reads of 16 consecutive rows (same
// k offset) must hit 16 distinct bank quads: with 128-byte rows the bank quad is (row parity, slot), hence lane
// (row r, slot v) fetches global vector v ^ ((r >> 1) & 7) and fragment reads apply the same XOR (no padding).
// The 16 copies of slice k+1 (or of the next vocabulary tile's first slice) are slotted between the 64 MFMAs of slice
// k, one per two MFMAs, and awaited at the slice boundary; fragments for the next 16-wide k-step are fetched from LDS
// while the current 16 MFMAs issue.
//
// The MFMA "A" operand is the WEIGHT tile and "B" the HIDDEN tile, so in the 32x32 accumulator layout a lane's column
// is a TOKEN and its 16 registers are 16 vocabulary entries: the online softmax over the vocabulary is then a
// per-lane reduction over 64 accumulator values per token (4 tokens per lane, 12 state registers), with one cross-lane
// and one cross-wave merge at the very end.  Each wave computes 128 vocab x 128 tokens = 4x4 MFMA tiles (256 fp32
// accumulators per lane, held in AGPRs).  Vocabulary ranges are split over workgroups (flash-decoding style) and
// merged by a small combine kernel; the target logit comes from a gather-dot kernel (one wave per token).
// The same pipeline drives the backward's recompute kernel, whose epilogue turns each accumulator block into the
// gradient w.r.t. the logits and stores it transposed in bf16, and the forward variant that keeps the bf16 logits.
//
// Workgroup -> (XCD, row block, vocab split) mapping: hardware places consecutive workgroup ids round-robin on the
// 8 XCDs; the 32 workgroups resident on one XCD are arranged as (32/S) row blocks x S vocab splits so that hidden
// tiles are shared by S workgroups and weight tiles by 32/S workgroups inside that XCD's L2.
#include <mutex>

#include "device_utils.h"
#include "lmhead_pipeline.h"
#include "relax_amd.h"

namespace relax_amd {

// STORE: also writes the logits, rounded to bf16, into l_t [vocab, l_stride] (token contiguous), and takes the softmax
// statistics from the rounded values (what the reference's bf16 F.linear hands to its fp32 log-softmax), so that a
// backward pass reading l_t sees exactly the distribution the forward pass normalised.
template <bool STORE, bool PAIRS>
__global__ __launch_bounds__(kLmThreads, 1) void lmhead_fwd_kernel(const uint16_t* __restrict__ hidden,
                                                                   const uint16_t* __restrict__ weight, LmGeom g,
                                                                   float c, float* __restrict__ partial,
                                                                   uint16_t* __restrict__ l_t, int64_t l_stride) {
  __shared__ __attribute__((aligned(1024))) unsigned char w0[kLmOperandBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char h0[kLmOperandBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char w1[kLmOperandBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char h1[kLmOperandBytes];
  unsigned char* smem = w0;
  int rb, split;
  if (!lm_block_coords(g, rb, split)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wv = wave >> 1, wt = wave & 1;
  const int64_t tok0 = int64_t(rb) * kLmTile;
  float m[4], s[4], t[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    m[j] = kNegHuge;
    s[j] = 0.f;
    t[j] = 0.f;
  }
  const int vt_begin = split * g.tiles_per_split;
  const int vt_end = min(g.n_tiles, vt_begin + g.tiles_per_split);
  LmSlabWriter writer;
  if (STORE) writer.init(l_t, l_stride, g.vocab, g.n_tokens, tok0, wv, wt, lane);
  lm_pipeline<STORE>(LmLds{w0, h0, w1, h1}, hidden, weight, g, tok0, vt_begin, vt_end, [&](floatx16 (&acc)[4][4], int64_t v0) {
    const int limit = int(min<int64_t>(g.vocab - v0, kLmTile));
    if (STORE) writer.set_tile(v0);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // one 16-value block at a time: without the barrier all 256 accumulators are copied out of the AGPRs first
        floatx16 blk = acc[i][j];
        if (STORE) {
          float x[16];
#pragma unroll
          for (int r = 0; r < 16; r += 2) {
            x[r] = blk[r];
            x[r + 1] = blk[r + 1];
            const uint32_t pk = pack_bf16(x[r], x[r + 1]);
            blk[r] = bf16_lo(pk);
            blk[r + 1] = bf16_hi(pk);
          }
          writer.template store<PAIRS>(x, i, j);
        }
        if (limit < kLmTile)  // ragged last tile: entries past the vocabulary are masked out
          lm_absorb_block<true>(blk, wv * 128 + i * 32 + 4 * (lane >> 5), limit, c, m[j], s[j], t[j]);
        else
          lm_absorb_block<false>(blk, 0, 0, c, m[j], s[j], t[j]);
        __builtin_amdgcn_sched_barrier(0);
      }
  });
  // merge the two lane halves (same tokens, different vocab rows), then the two waves sharing the tokens
  float* red = reinterpret_cast<float*>(smem);  // [2 (wv)][256 tokens][3]
  __syncthreads();
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float m2 = lane_xor<32>(m[j]), s2 = lane_xor<32>(s[j]), t2 = lane_xor<32>(t[j]);
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

// Target logit read back from the stored bf16 logits (so log_prob uses the very value the statistics saw).
__global__ __launch_bounds__(256) void lmhead_target_from_logits_kernel(const uint16_t* __restrict__ l_t,
                                                                        int64_t l_stride, int64_t n_tokens,
                                                                        int64_t vocab,
                                                                        const int64_t* __restrict__ targets,
                                                                        float* __restrict__ x_target) {
  const int64_t tok = blockIdx.x * 256LL + threadIdx.x;
  if (tok >= n_tokens) return;
  const int64_t tg = targets[tok];
  x_target[tok] = (tg < 0 || tg >= vocab) ? __builtin_nanf("") : bf16_lo(l_t[tg * l_stride + tok]);
}

// Backward from stored logits: overwrites l_t [vocab, stride] (bf16 logits, token contiguous) with the gradient
// dT[v, n] = inv_T * ( g_lp*(onehot - p) + g_H * p * (spx - x) ),  p = exp(x - lse)  -- the same expression the
// recomputing kernel evaluates on its accumulators.  A thread owns eight neighbouring tokens (one 16-byte access per
// vocabulary row) and keeps their per-token coefficients in registers while it walks `rows_per_block` rows.  Columns
// n_tokens .. ceil8(n_tokens) - 1 (the rest of the last 16-byte vector) are written as zeros, later ones not at all.
constexpr int kLmInplaceThreads = 256;
__global__ __launch_bounds__(kLmInplaceThreads) void lmhead_dlogits_inplace_kernel(
    uint16_t* __restrict__ l_t, int64_t stride, int64_t n_tokens, int64_t vocab, int rows_per_block, float c,
    float inv_t, const int64_t* __restrict__ targets, const float* __restrict__ lse, const float* __restrict__ spx,
    const float* __restrict__ g_lp, const float* __restrict__ g_ent, const float* __restrict__ grad_scale_dev) {
  const int64_t tok8 = (int64_t(blockIdx.x) * kLmInplaceThreads + threadIdx.x) * 8;
  if (tok8 >= n_tokens) return;
  const float gs = grad_scale_dev ? *grad_scale_dev : 1.0f;
  float k0[8], a0[8], a1[8], hot[8];
  int64_t tg[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int64_t tk = tok8 + k < n_tokens ? tok8 + k : n_tokens - 1;
    const float glp = g_lp[tk] * gs, gh = g_ent ? g_ent[tk] * gs : 0.f;
    const float b = gh * inv_t;
    k0[k] = -lse[tk] * kLog2e;
    a0[k] = -glp * inv_t + (g_ent ? b * spx[tk] : 0.f);
    a1[k] = -b * inv_t;
    hot[k] = glp * inv_t;
    tg[k] = tok8 + k < n_tokens ? targets[tk] : -1;
  }
  const int64_t v_begin = int64_t(blockIdx.y) * rows_per_block;
  const int64_t v_end = min<int64_t>(vocab, v_begin + rows_per_block);
  // four rows in flight per thread: the loads of a group are issued before its first store (in place, so the compiler
  // must not be asked to reorder them itself)
  for (int64_t v = v_begin; v < v_end; v += 4) {
    u32x4 raw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (v + u < v_end) raw[u] = *reinterpret_cast<const u32x4*>(l_t + (v + u) * stride + tok8);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (v + u >= v_end) break;
      float x[8], d[8];
      Row<bf16_t>::unpack(raw[u], x);
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        d[k] = fast_exp2(fmaf(x[k], c, k0[k])) * fmaf(x[k], a1[k], a0[k]);
        if (v + u == tg[k]) d[k] += hot[k];
        if (tok8 + k >= n_tokens) d[k] = 0.f;  // the vector's tail past the last token: padding, kept at zero
      }
      u32x4 o;
      o.x = pack_bf16(d[0], d[1]);
      o.y = pack_bf16(d[2], d[3]);
      o.z = pack_bf16(d[4], d[5]);
      o.w = pack_bf16(d[6], d[7]);
      *reinterpret_cast<u32x4*>(l_t + (v + u) * stride + tok8) = o;
    }
  }
}

// Backward helper: recompute one [chunk, V] slab of logits on the matrix cores and emit, transposed, the bf16
// gradient w.r.t. the logits  dT[v, n] = inv_T * ( g_lp*(onehot - p) + g_H * p * (spx - x) ),  p = exp(x - lse).
// dT is [vocab, chunk] (token-contiguous) so a lane's 32 neighbours write one 64-byte segment.
template <bool PAIRS>
__global__ __launch_bounds__(kLmThreads, 1) void lmhead_dlogits_kernel(
    const uint16_t* __restrict__ hidden, const uint16_t* __restrict__ weight, LmGeom g, float c, float inv_t,
    const int64_t* __restrict__ targets, const float* __restrict__ lse, const float* __restrict__ spx,
    const float* __restrict__ g_lp, const float* __restrict__ g_ent, const float* __restrict__ grad_scale_dev,
    uint16_t* __restrict__ d_t, int64_t d_stride) {
  __shared__ __attribute__((aligned(1024))) unsigned char w0[kLmOperandBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char h0[kLmOperandBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char w1[kLmOperandBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char h1[kLmOperandBytes];
  int rb, split;
  if (!lm_block_coords(g, rb, split)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wv = wave >> 1, wt = wave & 1;
  const int64_t tok0 = int64_t(rb) * kLmTile;
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
  LmSlabWriter writer;
  writer.init(d_t, d_stride, g.vocab, g.n_tokens, tok0, wv, wt, lane);
  lm_pipeline<true>(LmLds{w0, h0, w1, h1}, hidden, weight, g, tok0, vt_begin, vt_end, [&](floatx16 (&acc)[4][4], int64_t v0) {
    writer.set_tile(v0);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int64_t vb = v0 + wv * 128 + i * 32 + 4 * (lane >> 5);
        const floatx16 blk = acc[i][j];
        float d[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const float x = blk[r];
          d[r] = fast_exp2(fmaf(x, c, k0[j])) * fmaf(x, a1[j], a0[j]);
          if (vb + 8 * (r >> 2) + (r & 3) == tg[j]) d[r] += hot[j];
        }
        writer.template store<PAIRS>(d, i, j);
        __builtin_amdgcn_sched_barrier(0);
      }
  });
}

}  // namespace relax_amd

using namespace relax_amd;

static int lm_max_splits(int64_t n_tokens);

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
  if (hidden % (2 * kLmBK) != 0 || h_stride % 8 != 0 || w_stride % 8 != 0 || !aligned16(h) || !aligned16(w) ||
      int64_t(kLmTile) * h_stride >= (1LL << 31) || int64_t(kLmTile) * w_stride >= (1LL << 31)) {
    set_error("%s: hidden size must be a multiple of %d and rows 16-byte aligned (hidden=%lld)", what, 2 * kLmBK,
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
  int s = lm_max_splits(n);
  while (s > 1 && s > g.n_tiles) s /= 2;
  g.splits = s;
  g.tiles_per_split = (g.n_tiles + s - 1) / s;
  return RELAX_AMD_OK;
}

// Vocabulary splits per row block as far as the token count decides (the workspace is sized from it): enough to put
// two workgroups on every CU while that takes at most 8 splits, and for short inputs up to 32 (one row block per XCD)
// as long as fewer than 256 workgroups would otherwise have work.
static int lm_max_splits(int64_t n_tokens) {
  const int64_t row_blocks = (n_tokens + kLmTile - 1) / kLmTile;
  int s = 1;
  while (s < 8 && row_blocks * s < 512) s *= 2;
  while (s < kLmPerXcd && row_blocks * s < 256) s *= 2;
  return s;
}

// floats of per-split softmax partials in the workspace (three per token and split)
static int64_t lm_partial_floats(int64_t n_tokens) {
  const int s = lm_max_splits(n_tokens);
  return int64_t(s < 8 ? 8 : s) * 3 * n_tokens;
}

static unsigned lm_grid(const LmGeom& g) {
  const int rb_per_round = kLmXcds * (kLmPerXcd / g.splits);
  const int rounds = (g.row_blocks + rb_per_round - 1) / rb_per_round;
  return unsigned(rounds) * kLmXcds * kLmPerXcd;
}

extern "C" int64_t relax_amd_lmhead_workspace_bytes(int64_t n_tokens) {
  if (n_tokens <= 0) return 0;
  return (lm_partial_floats(n_tokens) + n_tokens) * int64_t(sizeof(float));
}

// 4-byte paired stores need an even row stride and a 4-byte aligned base
static bool lm_pairs_ok(const void* p, int64_t stride) {
  return stride % 2 == 0 && reinterpret_cast<uintptr_t>(p) % 4 == 0;
}
// the slab writer keeps byte offsets inside a 256-row tile in 32 bits
static int lm_slab_stride_ok(const char* what, int64_t stride) {
  if (int64_t(kLmTile + 1) * stride * 2 >= (1LL << 31)) {
    set_error("%s: slab row stride %lld too large", what, (long long)stride);
    return RELAX_AMD_EUNSUPPORTED;
  }
  return RELAX_AMD_OK;
}

static int lm_forward(const char* what, const void* hidden, const void* weight, int dtype, int64_t n_tokens,
                      int64_t hidden_size, int64_t vocab, int64_t h_stride, int64_t w_stride, const int64_t* targets,
                      float inv_temperature, void* workspace, float* log_prob, float* entropy, float* lse, float* spx,
                      uint16_t* l_t, int64_t l_stride, void* stream) {
  LmGeom g;
  if (int rc = lm_geometry(what, dtype, n_tokens, hidden_size, vocab, h_stride, w_stride, hidden, weight, g)) return rc;
  if (!targets || !workspace || !log_prob || !(inv_temperature > 0.f)) {
    set_error("%s: NULL argument or non-positive inv_temperature", what);
    return RELAX_AMD_EINVAL;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* partial = static_cast<float*>(workspace);
  float* x_target = partial + lm_partial_floats(n_tokens);
  const uint16_t* h = static_cast<const uint16_t*>(hidden);
  const uint16_t* w = static_cast<const uint16_t*>(weight);
  const float c = inv_temperature * kLog2e;
  const dim3 grid(lm_grid(g)), block(kLmThreads);
  if (!l_t) {
    hipLaunchKernelGGL(lmhead_target_logit_kernel, dim3(unsigned((n_tokens + 3) / 4)), dim3(256), 0, s, h, w, g,
                       targets, x_target);
    if (int rc = check_launch("lmhead_target_logit")) return rc;
    hipLaunchKernelGGL((lmhead_fwd_kernel<false, false>), grid, block, 0, s, h, w, g, c, partial, nullptr, int64_t(0));
  } else if (lm_pairs_ok(l_t, l_stride)) {
    hipLaunchKernelGGL((lmhead_fwd_kernel<true, true>), grid, block, 0, s, h, w, g, c, partial, l_t, l_stride);
  } else {
    hipLaunchKernelGGL((lmhead_fwd_kernel<true, false>), grid, block, 0, s, h, w, g, c, partial, l_t, l_stride);
  }
  if (int rc = check_launch("lmhead_fwd")) return rc;
  if (l_t) {
    hipLaunchKernelGGL(lmhead_target_from_logits_kernel, dim3(unsigned((n_tokens + 255) / 256)), dim3(256), 0, s, l_t,
                       l_stride, n_tokens, vocab, targets, x_target);
    if (int rc = check_launch("lmhead_target_from_logits")) return rc;
  }
  hipLaunchKernelGGL(lmhead_combine_kernel, dim3(unsigned((n_tokens + 255) / 256)), dim3(256), 0, s, partial, x_target,
                     n_tokens, g.splits, inv_temperature, log_prob, entropy, lse, spx);
  return check_launch("lmhead_combine");
}

extern "C" int relax_amd_lmhead_logprob_fwd(const void* hidden, const void* weight, int dtype, int64_t n_tokens,
                                            int64_t hidden_size, int64_t vocab, int64_t h_stride, int64_t w_stride,
                                            const int64_t* targets, float inv_temperature, void* workspace,
                                            float* log_prob, float* entropy, float* lse, float* spx, void* stream) {
  if (n_tokens == 0) return RELAX_AMD_OK;
  return lm_forward("lmhead_logprob_fwd", hidden, weight, dtype, n_tokens, hidden_size, vocab, h_stride, w_stride,
                    targets, inv_temperature, workspace, log_prob, entropy, lse, spx, nullptr, 0, stream);
}

// Scratch of the allocation-free entry point: the per-split softmax partials and the target logits of up to
// RELAX_AMD_LMHEAD_STATIC_MAX_TOKENS tokens.  One copy per GPU, held until the process ends.  The name is a host-side
// stand-in, not a device address: host code only ever uses the pointer hipGetSymbolAddress returns for the current
// device.
static __device__ __align__(256) float lm_static_scratch[RELAX_AMD_LMHEAD_STATIC_SCRATCH_BYTES / sizeof(float)];

namespace {
constexpr int kLmMaxDevices = 64;
std::mutex lm_static_mutex;
void* lm_static_ptr[kLmMaxDevices] = {};
}  // namespace

// The current device's copy of lm_static_scratch (looked up once per device, with that device current).
static int lm_static_workspace(const char* what, void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kLmMaxDevices) {
    set_error("%s: no usable current device (%s)", what, e == hipSuccess ? "index out of range" : hipGetErrorString(e));
    return RELAX_AMD_EINVAL;
  }
  std::lock_guard<std::mutex> lock(lm_static_mutex);
  if (!lm_static_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(lm_static_scratch));
    if (e != hipSuccess || !p) {
      set_error("%s: hipGetSymbolAddress failed on device %d: %s", what, dev, hipGetErrorString(e));
      return RELAX_AMD_ELAUNCH;
    }
    lm_static_ptr[dev] = p;
  }
  *out = lm_static_ptr[dev];
  return RELAX_AMD_OK;
}

extern "C" int relax_amd_lmhead_logprob_fwd_static(const void* hidden, const void* weight, int dtype,
                                                   int64_t n_tokens, int64_t hidden_size, int64_t vocab,
                                                   int64_t h_stride, int64_t w_stride, const int64_t* targets,
                                                   float inv_temperature, float* log_prob, float* entropy, float* lse,
                                                   float* spx, void* stream) {
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (n_tokens < 0 || n_tokens > RELAX_AMD_LMHEAD_STATIC_MAX_TOKENS ||
      relax_amd_lmhead_workspace_bytes(n_tokens) > int64_t(RELAX_AMD_LMHEAD_STATIC_SCRATCH_BYTES)) {
    set_error("lmhead_logprob_fwd_static: n_tokens=%lld is outside 0..%d, the size the built-in scratch holds; use "
              "relax_amd_lmhead_logprob_fwd with a caller workspace", (long long)n_tokens,
              RELAX_AMD_LMHEAD_STATIC_MAX_TOKENS);
    return RELAX_AMD_EUNSUPPORTED;
  }
  void* workspace = nullptr;
  if (int rc = lm_static_workspace("lmhead_logprob_fwd_static", &workspace)) return rc;
  // every partial and target logit the combine kernel reads is written by this call's own launches first, so the
  // contents a previous call left behind need no clearing
  return lm_forward("lmhead_logprob_fwd_static", hidden, weight, dtype, n_tokens, hidden_size, vocab, h_stride,
                    w_stride, targets, inv_temperature, workspace, log_prob, entropy, lse, spx, nullptr, 0, stream);
}

extern "C" int relax_amd_lmhead_logprob_fwd_keep(const void* hidden, const void* weight, int dtype, int64_t n_tokens,
                                                 int64_t hidden_size, int64_t vocab, int64_t h_stride,
                                                 int64_t w_stride, const int64_t* targets, float inv_temperature,
                                                 void* workspace, float* log_prob, float* entropy, float* lse,
                                                 float* spx, void* logits_t, int64_t l_stride, void* stream) {
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (!logits_t || l_stride < n_tokens) {
    set_error("lmhead_logprob_fwd_keep: NULL logits_t or l_stride < n_tokens");
    return RELAX_AMD_EINVAL;
  }
  if (int rc = lm_slab_stride_ok("lmhead_logprob_fwd_keep", l_stride)) return rc;
  return lm_forward("lmhead_logprob_fwd_keep", hidden, weight, dtype, n_tokens, hidden_size, vocab, h_stride,
                    w_stride, targets, inv_temperature, workspace, log_prob, entropy, lse, spx,
                    static_cast<uint16_t*>(logits_t), l_stride, stream);
}

extern "C" int relax_amd_lmhead_dlogits_from_logits_t(void* logits_t, int64_t n_tokens, int64_t vocab,
                                                      int64_t l_stride, const int64_t* targets, const float* lse,
                                                      const float* spx, const float* g_lp, const float* g_ent,
                                                      const float* grad_scale_dev, float inv_temperature,
                                                      void* stream) {
  if (n_tokens == 0 || vocab == 0) return RELAX_AMD_OK;
  if (n_tokens < 0 || vocab < 0 || !logits_t || !targets || !lse || !g_lp || (g_ent && !spx) ||
      !(inv_temperature > 0.f)) {
    set_error("lmhead_dlogits_from_logits_t: NULL argument, negative size or non-positive inv_temperature");
    return RELAX_AMD_EINVAL;
  }
  if (l_stride % 8 != 0 || l_stride < n_tokens || !aligned16(logits_t)) {
    set_error("lmhead_dlogits_from_logits_t: l_stride must be a multiple of 8 and >= n_tokens, base 16-byte aligned");
    return RELAX_AMD_EUNSUPPORTED;
  }
  constexpr int kRows = 64;
  const int64_t col_blocks = (n_tokens + 8LL * kLmInplaceThreads - 1) / (8LL * kLmInplaceThreads);
  const int64_t row_blocks = (vocab + kRows - 1) / kRows;
  if (row_blocks > 65535 || col_blocks > 2147483647LL) {
    set_error("lmhead_dlogits_from_logits_t: vocab=%lld too large", (long long)vocab);
    return RELAX_AMD_EUNSUPPORTED;
  }
  hipLaunchKernelGGL(lmhead_dlogits_inplace_kernel, dim3(unsigned(col_blocks), unsigned(row_blocks)),
                     dim3(kLmInplaceThreads), 0, static_cast<hipStream_t>(stream), static_cast<uint16_t*>(logits_t),
                     l_stride, n_tokens, vocab, kRows, inv_temperature * kLog2e, inv_temperature, targets, lse, spx,
                     g_lp, g_ent, grad_scale_dev);
  return check_launch("lmhead_dlogits_inplace");
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
  if (int rc = lm_slab_stride_ok("lmhead_dlogits_t", d_stride)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (lm_pairs_ok(d_t, d_stride))
    hipLaunchKernelGGL(lmhead_dlogits_kernel<true>, dim3(lm_grid(g)), dim3(kLmThreads), 0, s,
                       static_cast<const uint16_t*>(hidden), static_cast<const uint16_t*>(weight), g,
                       inv_temperature * kLog2e, inv_temperature, targets, lse, spx, g_lp, g_ent, grad_scale_dev,
                       static_cast<uint16_t*>(d_t), d_stride);
  else
    hipLaunchKernelGGL(lmhead_dlogits_kernel<false>, dim3(lm_grid(g)), dim3(kLmThreads), 0, s,
                       static_cast<const uint16_t*>(hidden), static_cast<const uint16_t*>(weight), g,
                       inv_temperature * kLog2e, inv_temperature, targets, lse, spx, g_lp, g_ent, grad_scale_dev,
                       static_cast<uint16_t*>(d_t), d_stride);
  return check_launch("lmhead_dlogits");
}
