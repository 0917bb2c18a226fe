// Backward GEMMs of the fused LM head on the forward kernel's LDS-ring / MFMA pipeline:
//   dhidden[n, h] = sum_v d_t[v, n] * weight[v, h]      (contraction over the vocabulary)
//   dweight[v, h] = sum_n d_t[v, n] * hidden[n, h]      (contraction over the tokens)
// where d_t [vocab, tokens] is the bf16 gradient slab the recompute kernel writes (token contiguous).  Autograd through
// F.linear in the deferred-LM-head branch, relax/backends/megatron/loss.py:391-419 and model.py:151-166.
//
// One kernel template computes C[a, b] = sum_k A(a, k) * B(b, k) for a 256 x 256 tile of C per workgroup (four waves,
// 128 x 128 each on v_mfma_f32_32x32x16_bf16), looping over the whole contraction in 32-wide slices through a
// four-stage LDS ring.  Each operand is stored either with the contraction index contiguous ([rows, K]: the layout
// the forward kernel's operands have) or with it outermost ([K, rows], rows contiguous): every operand of the two
// products above except d_t in dweight is of the second kind, and no transposed copy of anything is made.  A
// K-outermost slice is copied global -> LDS as it lies (32 k-rows of 512 bytes) and the MFMA fragments, which want 8
// consecutive k per lane, are read with the transposing LDS load (ds_read_b64_tr_b16: 16 lanes x 4 elements are
// exchanged so that each lane receives 4 consecutive k-rows of one column), two per fragment.  The 16-byte slot of
// column chunk c in k-row r is c ^ ((r & 3) << 2), which spreads the four k-rows one transposing read touches over
// distinct banks (measured: no bank conflicts).
//
// What bounds it: the board's power limit.  With every operand read served from cache the dhidden shape runs at
// 0.63 - 0.65 of the published bf16 peak; streaming the operands from memory (60 GB per launch cross the L2 <-> fabric
// boundary, the floor for 32 workgroups per XCD sharing 4 + 8 panels) costs both matrix-core cycles and clock and
// leaves 0.54 - 0.57.  The same loop on v_mfma_f32_16x16x32_bf16 (8 x 8 tiles per wave) was built and measured: the
// clock rises from 1.5 - 1.65 to 1.9 - 2.1 GHz, but a single wave per SIMD cannot issue its fragment reads, copies and
// address arithmetic between 16-cycle matrix instructions, the matrix cores idle a third of the time and the launch
// takes longer (31.9 / 39.2 ms against 28.6 / 30.0 ms).
//
// Reads beyond an operand's extent are clamped to its last row / chunk, never out of bounds; the products stay exact
// because d_t is zero-padded: the caller allocates it with ceil128(vocab) rows of ceil128(tokens) columns and zeros
// in the padding, so a clamped (finite) value of the other operand is always multiplied by zero.
#include "lmhead_pipeline.h"
#include "relax_amd.h"

namespace relax_amd {

typedef short v4i16 __attribute__((ext_vector_type(4)));
typedef short v8i16 __attribute__((ext_vector_type(8)));

struct GemmOperand {
  const uint16_t* p;
  int64_t stride;   // elements between consecutive rows of the stored matrix
  int64_t m_read;   // readable extent of the output-side index (a multiple of 8 for a K-outermost operand)
  int64_t k_read;   // readable extent of the contraction index
};

// ---- the contraction loop: a four-stage LDS ring of 32-wide k-slices
//
// Operands stream through the ring with no reuse in time: every slice of both tiles is new data, and the workgroups
// that share a panel inside an XCD ask for it at the same moment, so each slice is paid for at memory latency, not at
// L2 latency.  The ring therefore keeps three slices in flight (16 KB per operand and slice, 128 KB in all): the
// copies of slice s + 3 are issued while slice s is multiplied, and the wait at the top of slice s leaves the 16
// younger copies of slices s + 1 and s + 2 outstanding (vmcnt counts in order).
constexpr int kGemmBK = 32;                                  // contraction elements per ring slot
constexpr int kGemmStages = 4;
constexpr int kGemmSlotBytes = kLmTile * kGemmBK * 2;        // 16 KB per operand
constexpr int kGemmPasses = 4;                               // 16-byte copies per thread, operand and slice
// s_waitcnt: vmcnt = 16 (bits [15:14] = 1, [3:0] = 0), expcnt and lgkmcnt left at their maxima
constexpr int kGemmWaitOlderCopies = 0x4F70;

// Copier of a K-outermost operand slice: 32 k-rows x 256 columns, stored as it lies (512 bytes per k-row).  Thread t
// covers k-row t/32 of each 8-row pass and LDS slot t%32 of that row; it fetches column chunk
// (t%32) ^ ((k-row & 3) << 2), the same chunk in every pass.
struct GemmCopierKM {
  const unsigned char* base;  // element (k = 0, first column of the tile); wave-uniform
  uint32_t off_full[kGemmPasses], off_tail[kGemmPasses];  // byte offsets inside a full slice / inside the last one
  uint32_t stride_b;
  int tail_slice;  // the slice that holds the operand's last k-row

  __device__ __forceinline__ void init(const GemmOperand& op, int64_t m0) {
    const int slot = threadIdx.x & 31, r = (threadIdx.x >> 5) & 3;
    const int last_chunk = int((op.m_read - m0) / 8) - 1;
    const int chunk = min(slot ^ (r << 2), last_chunk);
    base = reinterpret_cast<const unsigned char*>(op.p + m0);
    stride_b = uint32_t(op.stride * 2);
    const int k_last = int(op.k_read - 1);
    tail_slice = k_last / kGemmBK;
    const int lim = k_last - tail_slice * kGemmBK;  // rows 0 .. lim of the last slice exist
#pragma unroll
    for (int p = 0; p < kGemmPasses; ++p) {
      const int krow = p * 8 + int(threadIdx.x >> 5);
      off_full[p] = uint32_t(krow) * stride_b + uint32_t(chunk) * 16u;
      off_tail[p] = uint32_t(min(krow, lim)) * stride_b + uint32_t(chunk) * 16u;
    }
  }
  __device__ __forceinline__ void issue_pass(unsigned char* tile, int kslice, int p) const {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // a slice wholly past the end re-fetches the last one (its product is zero through the other operand's padding);
    // in the last slice, k-rows past the end re-read the last row
    const bool tail = kslice >= tail_slice;
    const int k0 = min(kslice, tail_slice) * kGemmBK;
    uint64_t slice = reinterpret_cast<uint64_t>(base) + uint64_t(k0) * uint64_t(stride_b);
    asm volatile("" : "+s"(slice));
    uint32_t lane_off = tail ? off_tail[p] : off_full[p];
    asm volatile("" : "+v"(lane_off));
    const unsigned char* src = reinterpret_cast<const unsigned char*>(slice + uint64_t(lane_off));
    unsigned char* dst = tile + (p * 256 + wave * 64) * 16;  // wave-uniform; lane l lands at dst + 16*l
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src),
                                     (__attribute__((address_space(3))) void*)(dst), 16, 0, 0);
  }
};

// Copier of a K-contiguous operand slice: 256 rows x 32 k, 64 bytes per row.  Thread t covers row t/4 of each 64-row
// pass and LDS slot t%4; it fetches the row's 16-byte k-chunk (t%4) ^ ((row >> 2) & 3), which makes the fragment reads
// of 16 consecutive rows hit 16 distinct bank groups.  Rows past the operand's end re-read its last row.
struct GemmCopierKC {
  const unsigned char* base;
  uint32_t off[kGemmPasses];

  __device__ __forceinline__ void init(const GemmOperand& op, int64_t m0) {
    const int r = threadIdx.x >> 2, v = threadIdx.x & 3;
    base = reinterpret_cast<const unsigned char*>(op.p + m0 * op.stride);
    const int last = int(op.m_read - 1 - m0);
#pragma unroll
    for (int p = 0; p < kGemmPasses; ++p) {
      const int row = r + 64 * p;
      off[p] = uint32_t(min(row, last)) * uint32_t(op.stride * 2) + uint32_t((v ^ ((row >> 2) & 3)) * 16);
    }
  }
  __device__ __forceinline__ void issue_pass(unsigned char* tile, int kslice, int p) const {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    uint64_t slice = reinterpret_cast<uint64_t>(base) + uint64_t(kslice) * (kGemmBK * 2);
    asm volatile("" : "+s"(slice));
    uint32_t lane_off = off[p];
    asm volatile("" : "+v"(lane_off));
    const unsigned char* src = reinterpret_cast<const unsigned char*>(slice + uint64_t(lane_off));
    unsigned char* dst = tile + (p * 256 + wave * 64) * 16;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src),
                                     (__attribute__((address_space(3))) void*)(dst), 16, 0, 0);
  }
};

template <bool KM>
struct GemmCopier;
template <>
struct GemmCopier<true> : GemmCopierKM {};
template <>
struct GemmCopier<false> : GemmCopierKC {};

// Fragment reads of one operand for one wave (128 of the tile's 256 rows, starting at row `m_base`); ks = 0 or 1, the
// 16-wide k-step inside the slice.
// K-contiguous: one 16-byte read per 32-row fragment: row (lane & 31), k-chunk 2*ks + (lane >> 5).
// K-outermost: two transposing 8-byte reads per fragment; lane l = 32*hf + 16*g + i of the read for k-rows
// kb .. kb+3 points at k-row kb + i/4, columns 4*(i%4) .. +3 of the 16-column group g, and receives column i of that
// group at the four k-rows.
template <bool KM>
struct GemmFragReader;

template <>
struct GemmFragReader<false> {
  static constexpr int kReads = 4;
  uint32_t off[2];
  __device__ __forceinline__ void init(int lane, int m_base) {
    const int row = lane & 31;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
      off[ks] = uint32_t((m_base + row) * (kGemmBK * 2) + (((2 * ks + (lane >> 5)) ^ ((row >> 2) & 3)) * 16));
  }
  __device__ __forceinline__ void read(const unsigned char* tile, int ks, int n, v4i16 (&f)[4][2]) const {
    const v8i16 v = *reinterpret_cast<const v8i16*>(tile + off[ks] + n * 32 * (kGemmBK * 2));
    f[n][0] = __builtin_shufflevector(v, v, 0, 1, 2, 3);
    f[n][1] = __builtin_shufflevector(v, v, 4, 5, 6, 7);
  }
};

template <>
struct GemmFragReader<true> {
  static constexpr int kReads = 8;
  uint32_t off[4];
  __device__ __forceinline__ void init(int lane, int m_base) {
    const int i = lane & 15, g = (lane >> 4) & 1, hf = lane >> 5, r = i >> 2;
#pragma unroll
    for (int ms = 0; ms < 4; ++ms) {
      const int m = m_base + ms * 32 + g * 16 + 4 * (i & 3);
      const int slot = (m >> 3) ^ (r << 2);
      off[ms] = uint32_t((8 * hf + r) * 512 + slot * 16 + (m & 7) * 2);
    }
  }
  __device__ __forceinline__ void read(const unsigned char* tile, int ks, int n, v4i16 (&f)[4][2]) const {
    const int ms = n >> 1, q = n & 1;
    const unsigned char* p = tile + off[ms] + (ks * 16 + 4 * q) * 512;
    f[ms][q] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) v4i16*)(p));
  }
};

struct GemmFrags {
  v4i16 a[4][2], b[4][2];
};

__device__ __forceinline__ bf16x8 gemm_frag(const v4i16 (&h)[2]) {
  return __builtin_bit_cast(bf16x8, __builtin_shufflevector(h[0], h[1], 0, 1, 2, 3, 4, 5, 6, 7));
}

// 16 MFMAs (one 16-wide k-step of the wave's 128 x 128 block) with other work slotted in: `between(n)` is emitted
// right after MFMA n and pinned there.
template <typename Between>
__device__ __forceinline__ void gemm_mma_group(const GemmFrags& f, floatx16 (&acc)[4][4], Between&& between) {
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(gemm_frag(f.a[i]), gemm_frag(f.b[j]), acc[i][j], 0, 0, 0);
      between(i * 4 + j);
      __builtin_amdgcn_sched_barrier(0);
    }
}

// The ring: four slots per operand, each its own LDS object so that the compiler can prove that fragment reads from
// one slot never alias the copies in flight into the others.
struct GemmRing {
  unsigned char* a[kGemmStages];
  unsigned char* b[kGemmStages];
};

// "the copies of the slice about to be multiplied have landed" (the 16 younger ones may still be in flight), then the
// workgroup barrier: every wave sees the slice, and every wave has issued its last read of the slot refilled next.
// No memory fence: LDS is coherent inside the workgroup and the counter wait is the completion signal.
__device__ __forceinline__ void gemm_slice_sync() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(kGemmWaitOlderCopies);
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
}

// `init_acc(acc)` gives the accumulators their starting values (zeros, or the earlier partial sums of an accumulating
// product); it runs after the first three slices have been requested, so whatever it loads travels with them.
template <bool AKM, bool BKM, typename InitAcc>
__device__ __forceinline__ void gemm_pipeline(const GemmRing ring, const GemmOperand& A, const GemmOperand& B,
                                              int64_t a0, int64_t b0, int nk, floatx16 (&acc)[4][4],
                                              InitAcc&& init_acc) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wa = wave >> 1, wb = wave & 1;
  GemmCopier<AKM> ac;
  GemmCopier<BKM> bc;
  ac.init(A, a0);
  bc.init(B, b0);
  GemmFragReader<AKM> ar;
  GemmFragReader<BKM> br;
  ar.init(lane, wa * 128);
  br.init(lane, wb * 128);
  // LDS reads of one k-step's fragments, in the order the MFMAs want them (A fragment 0, the four B fragments, then
  // A fragments 1..3); a fragment takes one read (K-contiguous) or two (K-outermost).
  constexpr int kPerA = GemmFragReader<AKM>::kReads / 4, kPerB = GemmFragReader<BKM>::kReads / 4;
  constexpr int kReads = 4 * (kPerA + kPerB);
  auto read_one = [&](int st, int ks, int n, GemmFrags& f) {
    if (n < kPerA)
      ar.read(ring.a[st], ks, n, f.a);
    else if (n < kPerA + 4 * kPerB)
      br.read(ring.b[st], ks, n - kPerA, f.b);
    else if (n < kReads)
      ar.read(ring.a[st], ks, n - 4 * kPerB, f.a);
  };
  // after MFMA n of a group: two fragment reads (all issued 8 or more MFMAs ahead of their use) ...
  auto read = [&](int st, int ks, int n, GemmFrags& f) {
    read_one(st, ks, 2 * n, f);
    read_one(st, ks, 2 * n + 1, f);
  };
  // ... and in the second half of a group, where no reads are left, one of the 8 copies of the slice three ahead
  // after every other MFMA (copies 0..3 in a slice's first group, 4..7 in its second)
  auto copy = [&](int st, int kslice, int n, int half) {
    if (n >= 8 && (n & 1)) {
      const int c = half * 4 + ((n - 8) >> 1);
      if (c < kGemmPasses)
        ac.issue_pass(ring.a[st], kslice, c);
      else
        bc.issue_pass(ring.b[st], kslice, c - kGemmPasses);
    }
  };
  auto copy_all = [&](int st, int kslice) {
#pragma unroll
    for (int c = 0; c < kGemmPasses; ++c) ac.issue_pass(ring.a[st], kslice, c);
#pragma unroll
    for (int c = 0; c < kGemmPasses; ++c) bc.issue_pass(ring.b[st], kslice, c);
  };
  GemmFrags f0, f1;
  // one slice in the steady state: its slot is `st`; the slot of the slice before it is refilled with slice s + 3
  // (slices past the end re-fetch the last one into a slot nobody reads again: cheaper than a branch here, and it
  // keeps the count of copies in flight what the wait expects)
  auto step = [&](int st, int s) {
    gemm_slice_sync();
    const int refill = (st + 3) & 3, ahead = min(s + 3, nk - 1);
    gemm_mma_group(f1, acc, [&](int n) {  // the previous slice's second k-step
      read(st, 0, n, f0);
      copy(refill, ahead, n, 0);
    });
    gemm_mma_group(f0, acc, [&](int n) {
      read(st, 1, n, f1);
      copy(refill, ahead, n, 1);
    });
  };

  copy_all(0, 0);
  copy_all(1, 1);
  copy_all(2, 2);
  init_acc(acc);
  gemm_slice_sync();
#pragma unroll
  for (int n = 0; n < kReads; ++n) read_one(0, 0, n, f0);
  copy_all(3, min(3, nk - 1));
  gemm_mma_group(f0, acc, [&](int n) { read(0, 1, n, f1); });
  int s = 1;
  for (; s + 3 < nk; s += 4) {  // nk is a multiple of 4, so slice s lives in slot s % 4 = 1, 2, 3, 0
    step(1, s);
    step(2, s + 1);
    step(3, s + 2);
    step(0, s + 3);
  }
  step(1, s);
  step(2, s + 1);
  step(3, s + 2);
  gemm_mma_group(f1, acc, [](int) {});
  __builtin_amdgcn_s_waitcnt(kLmWaitCopies);  // the stray copies of the tail
}

enum { kGemmOutBf16 = 0, kGemmOutF32 = 1, kGemmOutF32Accumulate = 2 };

struct GemmTiling {
  int tiles_a, tiles_b, sa, sb, supers_b;
};

// Workgroup -> tile: consecutive workgroup ids go round-robin to the 8 XCDs; the 32 workgroups resident on one XCD
// form an sa x sb block of tiles, so that inside that XCD's L2 an A panel is shared by sb and a B panel by sa
// workgroups; neighbouring XCDs take neighbouring blocks along b (the same A panels, shared through the memory-side
// cache).
__device__ __forceinline__ bool gemm_tile_coords(const GemmTiling& t, int& ta, int& tb) {
  const int id = blockIdx.x;
  const int xcd = id % kLmXcds, slot = (id / kLmXcds) % kLmPerXcd, round = id / (kLmXcds * kLmPerXcd);
  const int super = round * kLmXcds + xcd;
  ta = (super / t.supers_b) * t.sa + slot / t.sb;
  tb = (super % t.supers_b) * t.sb + slot % t.sb;
  return ta < t.tiles_a && tb < t.tiles_b;
}

template <bool AKM, bool BKM, int OUT, bool PAIRS>
__global__ __launch_bounds__(kLmThreads, 1) void lmhead_gemm_kernel(GemmOperand A, GemmOperand B, int nk, void* c_out,
                                                                    int64_t c_stride, int64_t ma, int64_t mb,
                                                                    GemmTiling tiling) {
  __shared__ __attribute__((aligned(1024))) unsigned char a0s[kGemmSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char a1s[kGemmSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char a2s[kGemmSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char a3s[kGemmSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char b0s[kGemmSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char b1s[kGemmSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char b2s[kGemmSlotBytes];
  __shared__ __attribute__((aligned(1024))) unsigned char b3s[kGemmSlotBytes];
  int ta, tb;
  if (!gemm_tile_coords(tiling, ta, tb)) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, wa = wave >> 1, wb = wave & 1;
  const int64_t a0 = int64_t(ta) * kLmTile, b0 = int64_t(tb) * kLmTile;
  floatx16 acc[4][4];
  const GemmRing ring{{a0s, a1s, a2s, a3s}, {b0s, b1s, b2s, b3s}};
  if (OUT == kGemmOutF32Accumulate) {
    // the product is added to what c_out holds: the tile's earlier values are the accumulators' starting point, read
    // while the first slices of the operands are on their way, and the epilogue is a plain store
    const float* c = static_cast<const float*>(c_out);
    gemm_pipeline<AKM, BKM>(ring, A, B, a0, b0, nk, acc, [&](floatx16 (&acc_)[4][4]) {
      const int64_t bcol = b0 + wb * 128 + (lane & 31);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int64_t arow = a0 + wa * 128 + i * 32 + 4 * (lane >> 5);
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int64_t a = arow + 8 * (r >> 2) + (r & 3), b = bcol + j * 32;
            acc_[i][j][r] = (a < ma && b < mb) ? c[a * c_stride + b] : 0.f;
          }
      }
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(kLmWaitCopies);  // everything requested so far, the three slices included
      __builtin_amdgcn_sched_barrier(0);
    });
  } else {
    gemm_pipeline<AKM, BKM>(ring, A, B, a0, b0, nk, acc, [](floatx16 (&acc_)[4][4]) { lm_zero_acc(acc_); });
  }
  if (OUT == kGemmOutBf16) {
    LmSlabWriter writer;
    writer.init(static_cast<uint16_t*>(c_out), c_stride, ma, mb, b0, wa, wb, lane);
    writer.set_tile(a0);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const floatx16 blk = acc[i][j];
        float d[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) d[r] = blk[r];
        writer.template store<PAIRS>(d, i, j);
        __builtin_amdgcn_sched_barrier(0);
      }
  } else {
    float* c = static_cast<float*>(c_out);
    const int64_t bcol = b0 + wb * 128 + (lane & 31);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const floatx16 blk = acc[i][j];
        const int64_t b = bcol + j * 32;
        const int64_t arow = a0 + wa * 128 + i * 32 + 4 * (lane >> 5);
        if (b < mb) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int64_t a = arow + 8 * (r >> 2) + (r & 3);
            if (a < ma) c[a * c_stride + b] = blk[r];
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
  }
}

}  // namespace relax_amd

using namespace relax_amd;

static int64_t ceil128(int64_t x) { return (x + 127) / 128 * 128; }

static GemmTiling gemm_tiling(int64_t ma, int64_t mb) {
  GemmTiling t;
  t.tiles_a = int((ma + kLmTile - 1) / kLmTile);
  t.tiles_b = int((mb + kLmTile - 1) / kLmTile);
  t.sb = 1;
  while (t.sb < 8 && t.sb < t.tiles_b) t.sb *= 2;
  t.sa = kLmPerXcd / t.sb;
  t.supers_b = (t.tiles_b + t.sb - 1) / t.sb;
  return t;
}

static unsigned gemm_grid(const GemmTiling& t) {
  const int supers = ((t.tiles_a + t.sa - 1) / t.sa) * t.supers_b;
  return unsigned((supers + kLmXcds - 1) / kLmXcds) * kLmXcds * kLmPerXcd;
}

template <bool AKM, bool BKM>
static int gemm_launch(const char* what, const GemmOperand& A, const GemmOperand& B, int64_t k_pad, void* c,
                       int64_t c_stride, int64_t ma, int64_t mb, int out_mode, hipStream_t s) {
  const GemmTiling t = gemm_tiling(ma, mb);
  const dim3 grid(gemm_grid(t)), block(kLmThreads);
  const int nk = int(k_pad / kGemmBK);
  if (out_mode == RELAX_AMD_GEMM_OUT_BF16) {
    const bool pairs = c_stride % 2 == 0 && reinterpret_cast<uintptr_t>(c) % 4 == 0;
    if (pairs)
      hipLaunchKernelGGL((lmhead_gemm_kernel<AKM, BKM, kGemmOutBf16, true>), grid, block, 0, s, A, B, nk, c, c_stride,
                         ma, mb, t);
    else
      hipLaunchKernelGGL((lmhead_gemm_kernel<AKM, BKM, kGemmOutBf16, false>), grid, block, 0, s, A, B, nk, c, c_stride,
                         ma, mb, t);
  } else if (out_mode == RELAX_AMD_GEMM_OUT_F32) {
    hipLaunchKernelGGL((lmhead_gemm_kernel<AKM, BKM, kGemmOutF32, false>), grid, block, 0, s, A, B, nk, c, c_stride, ma,
                       mb, t);
  } else {
    hipLaunchKernelGGL((lmhead_gemm_kernel<AKM, BKM, kGemmOutF32Accumulate, false>), grid, block, 0, s, A, B, nk, c,
                       c_stride, ma, mb, t);
  }
  return check_launch(what);
}

// Shape rules shared by the two entry points.
static int gemm_check(const char* what, const void* d_t, int64_t d_stride, const void* other, int64_t o_stride,
                      int64_t n_tokens, int64_t hidden_size, int64_t vocab, const void* out, int64_t out_stride,
                      int out_mode) {
  if (!d_t || !other || !out || n_tokens <= 0 || hidden_size <= 0 || vocab <= 0 || n_tokens > (1LL << 30)) {
    set_error("%s: NULL argument or bad shape n_tokens=%lld hidden=%lld vocab=%lld", what, (long long)n_tokens,
              (long long)hidden_size, (long long)vocab);
    return RELAX_AMD_EINVAL;
  }
  if (out_mode != RELAX_AMD_GEMM_OUT_BF16 && out_mode != RELAX_AMD_GEMM_OUT_F32 &&
      out_mode != RELAX_AMD_GEMM_OUT_F32_ACCUMULATE) {
    set_error("%s: unknown out_mode %d", what, out_mode);
    return RELAX_AMD_EINVAL;
  }
  if (d_stride < ceil128(n_tokens) || d_stride % 8 != 0 || !aligned16(d_t)) {
    set_error("%s: d_t needs a 16-byte aligned base and a row stride that is a multiple of 8 and at least "
              "ceil128(n_tokens) = %lld (got %lld), zero-filled beyond n_tokens", what, (long long)ceil128(n_tokens),
              (long long)d_stride);
    return RELAX_AMD_EUNSUPPORTED;
  }
  if (hidden_size % 8 != 0 || o_stride < hidden_size || o_stride % 8 != 0 || !aligned16(other) ||
      out_stride < hidden_size) {
    set_error("%s: hidden size and row strides must be multiples of 8, bases 16-byte aligned (hidden=%lld)", what,
              (long long)hidden_size);
    return RELAX_AMD_EUNSUPPORTED;
  }
  // 32-bit byte offsets inside a tile: 256 rows (K-contiguous) or 64 k-rows (K-outermost) of any operand, and the
  // output tile
  const int64_t widest = d_stride > o_stride ? d_stride : o_stride;
  if (int64_t(kLmTile + 1) * widest * 2 >= (1LL << 31) || int64_t(kLmTile + 1) * out_stride * 4 >= (1LL << 31)) {
    set_error("%s: row stride too large", what);
    return RELAX_AMD_EUNSUPPORTED;
  }
  return RELAX_AMD_OK;
}

extern "C" int relax_amd_lmhead_dhidden(const void* d_t, int64_t d_rows, int64_t d_stride, const void* weight,
                                        int64_t w_stride, int64_t n_tokens, int64_t hidden_size, int64_t vocab,
                                        void* d_hidden, int64_t dh_stride, int out_mode, void* stream) {
  if (n_tokens == 0) return RELAX_AMD_OK;
  if (d_rows < ceil128(vocab)) {
    set_error("lmhead_dhidden: d_t must hold ceil128(vocab) = %lld rows (zeros beyond vocab), got %lld",
              (long long)ceil128(vocab), (long long)d_rows);
    return RELAX_AMD_EUNSUPPORTED;
  }
  if (int rc = gemm_check("lmhead_dhidden", d_t, d_stride, weight, w_stride, n_tokens, hidden_size, vocab, d_hidden,
                          dh_stride, out_mode))
    return rc;
  // C[a = token, b = hidden unit] = sum_{k = vocabulary entry} d_t[k, a] * weight[k, b]: both operands K-outermost
  const int64_t k_pad = ceil128(vocab);
  const GemmOperand A = {static_cast<const uint16_t*>(d_t), d_stride, ceil128(n_tokens), k_pad};
  const GemmOperand B = {static_cast<const uint16_t*>(weight), w_stride, hidden_size, vocab};
  return gemm_launch<true, true>("lmhead_dhidden", A, B, k_pad, d_hidden, dh_stride, n_tokens, hidden_size, out_mode,
                                 static_cast<hipStream_t>(stream));
}

extern "C" int relax_amd_lmhead_dweight(const void* d_t, int64_t d_stride, const void* hidden, int64_t h_stride,
                                        int64_t n_tokens, int64_t hidden_size, int64_t vocab, void* d_weight,
                                        int64_t dw_stride, int out_mode, void* stream) {
  if (vocab == 0) return RELAX_AMD_OK;
  if (n_tokens == 0) {
    set_error("lmhead_dweight: n_tokens == 0 (nothing to contract; clear d_weight on the caller's side)");
    return RELAX_AMD_EINVAL;
  }
  if (int rc = gemm_check("lmhead_dweight", d_t, d_stride, hidden, h_stride, n_tokens, hidden_size, vocab, d_weight,
                          dw_stride, out_mode))
    return rc;
  // C[a = vocabulary entry, b = hidden unit] = sum_{k = token} d_t[a, k] * hidden[k, b]: A K-contiguous (rows of the
  // slab), B K-outermost
  const int64_t k_pad = ceil128(n_tokens);
  const GemmOperand A = {static_cast<const uint16_t*>(d_t), d_stride, vocab, k_pad};
  const GemmOperand B = {static_cast<const uint16_t*>(hidden), h_stride, hidden_size, n_tokens};
  return gemm_launch<false, true>("lmhead_dweight", A, B, k_pad, d_weight, dw_stride, vocab, hidden_size, out_mode,
                                  static_cast<hipStream_t>(stream));
}
