// Shared device code of the LM-head matrix-core kernels (forward, backward recompute, backward GEMMs): the
// global -> LDS copier, the swizzled fragment reads, the MFMA slice schedule, the (tile, k-slice) software pipeline and
// the transposed bf16 tile writer.  Layout and schedule are described at the top of lmhead.hip.
#ifndef RELAX_AMD_LMHEAD_PIPELINE_H
#define RELAX_AMD_LMHEAD_PIPELINE_H

#include "device_utils.h"

namespace relax_amd {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kLmTile = 256;                 // tokens per workgroup == vocab entries per tile
constexpr int kLmBK = 64;                    // hidden-size slice per pipeline stage (128 B per row)
constexpr int kLmThreads = 256;
constexpr int kLmPasses = 8;                 // 16-byte copies per thread per operand slice (32 rows per pass)
constexpr int kLmOperandBytes = kLmTile * kLmBK * 2;   // 32 KB
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

// s_waitcnt immediates, issued through the builtin so that the compiler's own wait-count bookkeeping sees them:
// "all vector-memory operations done" (vmcnt = 0, expcnt and lgkmcnt left at their maxima), and vmcnt = lgkmcnt = 0.
constexpr int kLmWaitCopies = 0x0F70;
constexpr int kLmWaitEverything = 0x0070;
constexpr int kLmWaitLdsAndScalar = 0xC07F;  // lgkmcnt = 0, vmcnt left at its maximum

// Asynchronous global -> LDS copy of one 256-row x 64-col bf16 slice of an operand.  Thread t covers row t/8 of each
// 32-row pass and LDS slot t%8; it fetches global vector (t%8) ^ ((row >> 1) & 7) of that row (the same value for
// every pass).  Rows past the ragged edge re-read the last valid row; their results are discarded by the caller.
struct LmCopier {
  const unsigned char* base;  // first row of the tile (wave-uniform, lives in scalar registers)
  uint32_t off[kLmPasses];    // byte offset of this thread's vector in each pass, k-slice 0

  __device__ __forceinline__ void init(const uint16_t* matrix, int64_t stride, int64_t row0, int64_t row_limit) {
    const int r = threadIdx.x >> 3, v = threadIdx.x & 7;
    base = reinterpret_cast<const unsigned char*>(matrix + row0 * stride);
    const int last = int(row_limit - row0);
    const uint32_t col = uint32_t((v ^ ((r >> 1) & 7)) * 16);
#pragma unroll
    for (int p = 0; p < kLmPasses; ++p) off[p] = uint32_t(min(r + 32 * p, last)) * uint32_t(stride * 2) + col;
  }
  // `tile` = LDS address of this operand's tile in the target stage.  The source address is a scalar base plus a
  // 32-bit per-lane offset, so each copy needs one address register instead of a 64-bit pair.
  __device__ __forceinline__ void issue_pass(unsigned char* tile, int kslice, int p) const {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint64_t slice = reinterpret_cast<uint64_t>(base) + uint64_t(kslice) * (kLmBK * 2);
    asm volatile("" : "+s"(slice));  // keep scalar base + 32-bit lane offset apart (no hoisted 64-bit lane addresses)
    uint32_t lane_off = off[p];
    asm volatile("" : "+v"(lane_off));  // widen next to the copy so it folds into the scalar-base address form
    const unsigned char* src = reinterpret_cast<const unsigned char*>(slice + uint64_t(lane_off));
    unsigned char* dst = tile + (p * 32 + wave * 8) * (kLmBK * 2);  // wave-uniform; lane l lands at dst + 16*l
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src),
                                     (__attribute__((address_space(3))) void*)(dst), 16, 0, 0);
  }
  __device__ __forceinline__ void issue(unsigned char* tile, int kslice) const {
#pragma unroll
    for (int p = 0; p < kLmPasses; ++p) issue_pass(tile, kslice, p);
  }
};

// LDS byte offset (inside an operand tile) of the fragment this lane feeds to the MFMA for 16-wide k-step `ks`:
// row (lane & 31) of a 32-row sub-tile, global vector 2*ks + (lane >> 5), stored at slot vector ^ ((row >> 1) & 7).
__device__ __forceinline__ int lm_frag_offset(int lane, int ks) {
  const int row = lane & 31;
  return row * (kLmBK * 2) + (((2 * ks + (lane >> 5)) ^ ((row >> 1) & 7)) * 16);
}

// Operands of the 16 MFMAs of one 16-wide k-step: four 32-row weight fragments and four 32-row hidden fragments.
struct LmFrags {
  bf16x8 a[4], b[4];
};

// One pipeline stage in LDS (a 64-wide k-slice of both operands) as seen by one wave: its 128 weight rows and its
// 128 hidden rows.
struct LmStage {
  const unsigned char* w;
  const unsigned char* h;
};

// LDS read number n (0..7) of the fragment set of k-step `ks`: weight fragments first, then hidden fragments.
__device__ __forceinline__ void lm_load_frag(const LmStage& st, int lane, int ks, int n, LmFrags& f) {
  const int fo = lm_frag_offset(lane, ks);
  if (n < 4)
    f.a[n] = *reinterpret_cast<const bf16x8*>(st.w + n * 32 * (kLmBK * 2) + fo);
  else
    f.b[n - 4] = *reinterpret_cast<const bf16x8*>(st.h + (n - 4) * 32 * (kLmBK * 2) + fo);
}

// The 16 MFMAs of one k-step with other work slotted in between: `between(n)` is emitted right after MFMA n, so LDS
// reads and global -> LDS copies issue in the shadow of the 8-pass matrix instructions instead of in front of them.
// The scheduling barriers pin that order (the compiler would otherwise sink every fragment read next to its use).
template <typename Between>
__device__ __forceinline__ void lm_mma_group(const LmFrags& f, floatx16 (&acc)[4][4], Between&& between) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.a[i], f.b[j], acc[i][j], 0, 0, 0);
      between(i * 4 + j);
      __builtin_amdgcn_sched_barrier(0);
    }
}

// The 16 copies of the following slice are spread over the slice's MFMAs, one copy per kLmCopyEvery MFMAs: four
// waves issuing one 1 KB copy per MFMA ask for twice what the vector-memory path accepts and stall at issue.
constexpr int kLmCopyEvery = 2;
template <typename Copy>
__device__ __forceinline__ void lm_copy_slot(int m, Copy&& copy) {  // m = index of the MFMA just issued, 0..63
  if (m % kLmCopyEvery == kLmCopyEvery - 1 && m / kLmCopyEvery < 16) copy(m / kLmCopyEvery);
}

// k-steps 0..2 of the slice in `st`; on entry f0 holds (or is receiving) the fragments of k-step 0, on exit f1 those
// of k-step 3, whose MFMAs are left to the caller: they run after the next barrier and cover the LDS latency of the
// next slice's first fragments.
template <typename Copy>
__device__ __forceinline__ void lm_slice_body(const LmStage& st, int lane, LmFrags& f0, LmFrags& f1,
                                              floatx16 (&acc)[4][4], Copy&& copy) {
  lm_mma_group(f0, acc, [&](int n) {
    if (n < 8) lm_load_frag(st, lane, 1, n, f1);
    lm_copy_slot(16 + n, copy);
  });
  lm_mma_group(f1, acc, [&](int n) {
    if (n < 8) lm_load_frag(st, lane, 2, n, f0);
    lm_copy_slot(32 + n, copy);
  });
  lm_mma_group(f0, acc, [&](int n) {
    if (n < 8) lm_load_frag(st, lane, 3, n, f1);
    lm_copy_slot(48 + n, copy);
  });
}

// The previous slice's last k-step (fragments in f1) while the fragments of k-step 0 of the slice in `st` load into
// f0; `copy(n)`, n = 0..15, issues the n-th global -> LDS copy of the slice after it.
template <typename Copy>
__device__ __forceinline__ void lm_slice_head(const LmStage& st, int lane, LmFrags& f0, const LmFrags& f1,
                                              floatx16 (&acc)[4][4], Copy&& copy) {
  lm_mma_group(f1, acc, [&](int n) {
    if (n < 8) lm_load_frag(st, lane, 0, n, f0);
    lm_copy_slot(n, copy);
  });
}

__device__ __forceinline__ void lm_zero_acc(floatx16 (&acc)[4][4]) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
}

// "my copies have landed" + workgroup barrier: after it the slice copied last is visible to every wave and every wave
// has finished reading the stage that is overwritten next.
__device__ __forceinline__ void lm_slice_sync() {
  __builtin_amdgcn_s_waitcnt(kLmWaitCopies);
  __syncthreads();
}

// Walks the vocabulary tiles [vt_begin, vt_end) of one 256-token row block as a single software pipeline over
// (tile, k-slice) and hands every finished 256x256 logits tile (fp32, un-scaled) to `epilogue(acc, v0)`, which runs
// while the first slice of the next tile is already in flight.
// Per slice and wave: barrier, then 64 MFMAs with the 32 fragment reads and the 16 copies of the following slice
// slotted between them.  The slice's last k-step is multiplied after the next barrier, so that barrier's wake-up
// and the first fragment reads of the new slice are covered by 16 MFMAs already in registers.
// The four operand tiles of the two-stage ring are distinct LDS objects (not regions of one buffer) so that the
// compiler can prove that fragment reads from one stage never alias the in-flight copies into the other; otherwise
// it waits for the copies before every LDS read and the overlap is lost.
struct LmLds {
  unsigned char *w0, *h0, *w1, *h1;  // weight / hidden tile of stage 0 and of stage 1
};

//
// EPILOGUE_STORES: the epilogue writes its tile to global memory (the kept logits, the gradient slab).  Vector-memory
// operations retire in order, so a wait for the next slice's copies issued after those stores would also wait until
// every store has been acknowledged by memory, once per tile.  In this form the copies of the next tile's first slice
// (issued under the last slice, i.e. before the stores) are awaited before the epilogue instead, the tile boundary is
// a bare barrier, and the stores drain under the next tile's first slice, whose closing wait finds them done.
template <bool EPILOGUE_STORES = false, typename Epilogue>
__device__ __forceinline__ void lm_pipeline(const LmLds lds, const uint16_t* hidden, const uint16_t* weight,
                                            const LmGeom& g, int64_t tok0, int vt_begin, int vt_end,
                                            Epilogue&& epilogue) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wv = wave >> 1, wt = wave & 1;
  const int nk = int(g.hidden / kLmBK);  // even: the hidden size is a multiple of 2 * kLmBK
  const LmStage st0 = {lds.w0 + wv * 128 * (kLmBK * 2), lds.h0 + wt * 128 * (kLmBK * 2)};
  const LmStage st1 = {lds.w1 + wv * 128 * (kLmBK * 2), lds.h1 + wt * 128 * (kLmBK * 2)};
  LmCopier hc, wc;
  hc.init(hidden, g.h_stride, tok0, g.n_tokens - 1);
  floatx16 acc[4][4];
  lm_zero_acc(acc);
  if (vt_begin >= vt_end) return;
  wc.init(weight, g.w_stride, int64_t(vt_begin) * kLmTile, g.vocab - 1);
  wc.issue(lds.w0, 0);
  hc.issue(lds.h0, 0);
  lm_slice_sync();
  LmFrags f0, f1;
  for (int vt = vt_begin; vt < vt_end; ++vt) {
    // Settle register reloads left over from the epilogue here, once per tile; otherwise the compiler waits for them
    // at their first use inside the steady-state loop, which also drains the copies issued just before.
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(EPILOGUE_STORES ? kLmWaitLdsAndScalar : kLmWaitEverything);
    __builtin_amdgcn_sched_barrier(0);
    // slice 0 (stage 0): nothing to multiply yet, so its first fragments are waited for in the open
#pragma unroll
    for (int n = 0; n < 8; ++n) lm_load_frag(st0, lane, 0, n, f0);
    wc.issue(lds.w1, 1);
    hc.issue(lds.h1, 1);
    __builtin_amdgcn_sched_barrier(0);
    lm_slice_body(st0, lane, f0, f1, acc, [](int) {});
    lm_slice_sync();
    for (int s = 1; s + 1 < nk; s += 2) {  // odd slices live in stage 1, even slices in stage 0
      auto copy_to_0 = [&](int n) {
        if (n < 8) {
          wc.issue_pass(lds.w0, s + 1, n);
        } else {
          hc.issue_pass(lds.h0, s + 1, n - 8);
        }
      };
      auto copy_to_1 = [&](int n) {
        if (n < 8) {
          wc.issue_pass(lds.w1, s + 2, n);
        } else {
          hc.issue_pass(lds.h1, s + 2, n - 8);
        }
      };
      lm_slice_head(st1, lane, f0, f1, acc, copy_to_0);
      lm_slice_body(st1, lane, f0, f1, acc, copy_to_0);
      lm_slice_sync();
      lm_slice_head(st0, lane, f0, f1, acc, copy_to_1);
      lm_slice_body(st0, lane, f0, f1, acc, copy_to_1);
      lm_slice_sync();
    }
    // Last slice of the tile (stage 1).  The copies issued under it fetch the next tile's first slice; after the last
    // tile they re-fetch this tile's first slice, which nobody reads (cheaper than a branch between the MFMAs).
    if (vt + 1 < vt_end) wc.init(weight, g.w_stride, int64_t(vt + 1) * kLmTile, g.vocab - 1);
    auto copy_next_tile = [&](int n) {
      if (n < 8) {
        wc.issue_pass(lds.w0, 0, n);
      } else {
        hc.issue_pass(lds.h0, 0, n - 8);
      }
    };
    lm_slice_head(st1, lane, f0, f1, acc, copy_next_tile);
    lm_slice_body(st1, lane, f0, f1, acc, copy_next_tile);
    lm_mma_group(f1, acc, [](int) {});
    if (EPILOGUE_STORES) {
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(kLmWaitCopies);  // the next tile's first slice: issued a slice ago, before any store
      __builtin_amdgcn_sched_barrier(0);
    }
    epilogue(acc, int64_t(vt) * kLmTile);
    lm_zero_acc(acc);
    if (EPILOGUE_STORES) {
      // every wave has passed its own wait above, so all copies into stage 0 have landed, and every wave is done
      // reading stage 1; no wait for the stores
      __builtin_amdgcn_sched_barrier(0);
      asm volatile("s_barrier" ::: "memory");
      __builtin_amdgcn_sched_barrier(0);
    } else {
      lm_slice_sync();
    }
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

// Writes accumulator blocks, as bf16, into a [vocab, token] matrix (token contiguous).  Addresses are a wave-uniform
// tile base plus one 32-bit lane offset plus a uniform per-store offset, so the 256 stores of a tile cost one vector
// add each and no 64-bit lane arithmetic.  Neighbouring lanes hold neighbouring tokens of the same vocabulary rows:
// with PAIRS an even/odd lane pair swaps one value per two rows and each lane writes two tokens with one 4-byte store,
// half the store instructions of the 2-byte form (needs an even row stride and a 4-byte aligned matrix).  Tiles that
// cross the end of the vocabulary or of the tokens take a checked 2-byte path.
struct LmSlabWriter {
  uint16_t* matrix;
  int64_t stride, vocab, n_tokens, tok0;
  unsigned char* tile;  // element (v0, tok0) of the current tile
  int64_t v0;
  uint32_t lane_off, lane_off_pair, stride_b;
  int wv, wt, lane;
  bool interior;

  __device__ __forceinline__ void init(uint16_t* m, int64_t stride_, int64_t vocab_, int64_t n_tokens_, int64_t tok0_,
                                       int wv_, int wt_, int lane_) {
    matrix = m, stride = stride_, vocab = vocab_, n_tokens = n_tokens_, tok0 = tok0_;
    wv = wv_, wt = wt_, lane = lane_;
    stride_b = uint32_t(stride * 2);
    const uint32_t row = uint32_t(wv * 128 + 4 * (lane >> 5)), col = uint32_t(wt * 128 + (lane & 31));
    lane_off = row * stride_b + col * 2;
    lane_off_pair = (row + (lane & 1)) * stride_b + (col & ~1u) * 2;
  }
  __device__ __forceinline__ void set_tile(int64_t v0_) {
    v0 = v0_;
    tile = reinterpret_cast<unsigned char*>(matrix + v0 * stride + tok0);
    interior = v0 + kLmTile <= vocab && tok0 + kLmTile <= n_tokens;
  }
  // block (i, j) of the wave's 4 x 4 accumulator blocks; d[r] = value of accumulator register r
  template <bool PAIRS>
  __device__ __forceinline__ void store(const float (&d)[16], int i, int j) const {
    using gptr32 = __attribute__((address_space(1))) uint32_t*;
    using gptr16 = __attribute__((address_space(1))) uint16_t*;
    if (interior) {
      uint64_t base = reinterpret_cast<uint64_t>(tile);
      asm volatile("" : "+s"(base));
      const uint32_t block_off = uint32_t(i * 32) * stride_b + uint32_t(j * 64);
      if (PAIRS) {
        uint32_t lo = lane_off_pair;
        asm volatile("" : "+v"(lo));
        const bool odd = lane & 1;
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const float send = odd ? d[2 * q] : d[2 * q + 1];
          // quad_perm [1, 0, 3, 2]: exchange with the neighbouring lane
          const float recv =
              __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(send), 0xB1, 0xF, 0xF, true));
          const uint32_t word = odd ? pack_bf16(recv, d[2 * q + 1]) : pack_bf16(d[2 * q], recv);
          const uint32_t row_even = uint32_t(8 * ((2 * q) >> 2) + ((2 * q) & 3));
          *(gptr32)(base + uint64_t(lo + (block_off + row_even * stride_b))) = word;
        }
      } else {
        uint32_t lo = lane_off;
        asm volatile("" : "+v"(lo));
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          const uint32_t pk = pack_bf16(d[r], d[r + 1]);
          const uint32_t row = uint32_t(8 * (r >> 2) + (r & 3));
          *(gptr16)(base + uint64_t(lo + (block_off + row * stride_b))) = uint16_t(pk);
          *(gptr16)(base + uint64_t(lo + (block_off + (row + 1) * stride_b))) = uint16_t(pk >> 16);
        }
      }
    } else {
      const int64_t tok = tok0 + wt * 128 + j * 32 + (lane & 31);
      const int64_t vb = v0 + wv * 128 + i * 32 + 4 * (lane >> 5);
      if (tok < n_tokens) {
        uint16_t* p = matrix + vb * stride + tok;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = 8 * (r >> 2) + (r & 3);
          if (vb + row < vocab) p[row * stride] = uint16_t(f32_to_bf16_bits(d[r]));
        }
      }
    }
  }
};

}  // namespace relax_amd

#endif  // RELAX_AMD_LMHEAD_PIPELINE_H
