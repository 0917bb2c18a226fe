// Register-resident fused actor step: the same computation as actor_step_fused_kernel (log-prob + entropy forward,
// per-token policy-loss coefficients, dlogits backward, one launch) for long 16-bit rows of the common vocabulary sizes
// and for fp32 rows of 32000 entries (and a few neighbouring sizes of either kind, see the launcher).
//
// A 1024-thread workgroup holds a whole row in its vector registers (V = 151936 bf16 is 18992 16-byte vectors = 19 per
// thread = 76 registers), so HBM sees exactly one read and one write per row and the second walk over the row costs no
// cache or fabric traffic at all.  One such workgroup fits a CU (fp32 rows of 32000 entries: 8 vectors per thread); the
// workgroups are persistent (one per CU, rows b, b + grid, ...) and take a row in three steps: the resident row becomes its gradient in place; the gradient leaves in
// one burst of stores and, into the registers those free, the workgroup's next live row arrives in one burst of loads
// (304 KB out, 304 KB in, each contiguous); the new row's softmax scan follows its loads in their order.  Memory rewards
// the long bursts: with a store and a load alternating vector by vector (and the scan trailing four vectors behind) the
// launch took 6.95 - 7.05 ms on the 65536 x 151936 workload, in blocks of 4 / 8 / 12 vectors 6.77 / 6.63 / 6.57 ms, a
// whole row at a time 6.49 ms, although nothing of one workgroup's arithmetic overlaps its own memory traffic any more
// (other CUs' bursts fill the gaps).  No workgroup waits for another; the loop bound is the only exit condition.
//
// The number of vectors per thread is a template parameter (full vector positions NVF, plus one partially filled
// position when PARTIAL), so the store / load loop is straight-line code without per-lane bounds checks.  That matters
// for more than instruction count: the compiler can only count how many loads and stores may stay in flight at each
// later use when no branch separates them; behind bounds checks it waits for all of them, stores included, several times
// per row.  Row lengths without an instantiation take the two-walk kernel.
//
// The scan over the registers repeats scan_row()'s grouping and order exactly (four vectors absorbed together while a
// thread has four to go, then single vectors; waves merged in index order), so log-probs stay bit-identical to the
// forward-only kernel's, which Relax's step-0 check (ppo_kl == 0 for identical weights) relies on.
//
// Replaces, like the two-walk kernel, _VocabParallelLogProbEntropy.forward + .backward
// (relax/utils/training/ppo_utils.py:481-629) and the per-token part of policy_loss_function
// (relax/backends/megatron/loss.py:961-1100) for one micro-batch.
//
// The kernels sit at the edge of the register file (76 of 128 registers hold the row).  With the scheduler's generic
// register-pressure tracking the allocator ends up parking parts of the row in scratch memory; with the AMDGPU
// trackers it does not:
// hipcc-flags: -mllvm -amdgpu-use-amdgpu-trackers=1
#include "actor_step_resident.h"

#include "device_utils.h"
#include "loss_math.h"
#include "opd_topk_math.h"
#include "row_scan.h"

namespace relax_amd {

// scan_absorb() over the values of kScanUnroll raw vectors, without holding them all unpacked
template <typename T>
__device__ __forceinline__ void absorb_raw_group(const u32x4* raw, float c, SoftmaxAcc& st) {
  constexpr int VN = Row<T>::kPerVec;
  float vmax = 0.f;
#pragma unroll
  for (int u = 0; u < kScanUnroll; ++u) {
    float v[VN];
    Row<T>::unpack(raw[u], v);
#pragma unroll
    for (int k = 0; k < VN; ++k) vmax = (u == 0 && k == 0) ? v[0] : fmaxf(vmax, v[k]);
    __builtin_amdgcn_sched_barrier(0);  // one vector's worth of temporaries at a time (see the callers)
  }
  const float mc = __fmul_rn(vmax, c);
  if (mc > st.m) {
    const float sc = fast_exp2(fmaf(-vmax, c, st.m));  // one rounding, spelled out (see scan_finish)
    st.s = __fmul_rn(st.s, sc);
    st.t = __fmul_rn(st.t, sc);
    st.m = mc;
  }
#pragma unroll
  for (int u = 0; u < kScanUnroll; ++u) {
    // unpack again from an opaque copy of the raw vector: the 32 values of the first walk kept alive (which is what
    // common-subexpression elimination would do) do not fit the register file next to the resident row
    u32x4 r = raw[u];
    asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
    float v[VN];
    Row<T>::unpack(r, v);
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      const float e = fast_exp2(fmaf(v[k], c, -st.m));
      st.s = __fadd_rn(st.s, e);
      st.t = fmaf(e, v[k], st.t);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// What thread 0 needs of a token before it can evaluate the loss terms.
struct ResidentTokenData {
  TokenInputs in;
  float x_target, den, pg_den;
  int64_t tg;
};

// Workgroup width: one 1024-thread workgroup per CU for every element type.  (fp32 rows of 32000 entries used to run
// in two 512-thread workgroups per CU with 16 vectors per thread; a plain stream of such rows in that arrangement
// moves 5.39 TB/s, in this one 5.62: a CU's stores and loads leave in longer runs of one kind.)
template <typename T>
constexpr int resident_threads() {
  return 1024;
}

template <typename T, int NVF, bool PARTIAL, bool TOPK = false>
__global__ __launch_bounds__(resident_threads<T>(), 4) void actor_step_resident_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
    const int32_t* __restrict__ token_of_row, const int32_t* __restrict__ sample_ids,
    const int64_t* __restrict__ targets, float c, float inv_t, relax_amd_policy_loss_args a, float grad_scale,
    float* __restrict__ log_prob, float* __restrict__ entropy, float* __restrict__ lse_out,
    float* __restrict__ spx_out, T* __restrict__ dlogits, int64_t d_stride) {
  constexpr int THREADS = resident_threads<T>(), kU = kScanUnroll;
  constexpr int VN = Row<T>::kPerVec;
  constexpr int NV = NVF + (PARTIAL ? 1 : 0);  // vector positions per thread
  constexpr int kGroups = (NV + kU - 1) / kU;
  __shared__ float wave_state[THREADS / kWave][3];
  __shared__ float bc[5];
  __shared__ int64_t bc_target;
  __shared__ float topk_stage[TOPK ? kTopkStageFloats : 1];
  const int tid = threadIdx.x;
  const bool wave0 = __builtin_amdgcn_readfirstlane(tid) < kWave;  // scalar: other waves branch around thread 0's work
  const int rem = int(vocab / VN) - NVF * THREADS;  // lanes that hold a vector at the partial position (host-checked)
  u32x4 reg[NV];

  // does this lane hold a vector at position j?  A compile-time answer except at the partial position.
  auto has = [&](int j) -> bool { return j < NVF || (PARTIAL && j == NVF && tid < rem); };

  // token of a row, or -1 when the row scores nothing or both of its masks are zero (uniform over the workgroup)
  auto live_token = [&](int64_t row) -> int64_t {
    if (row >= n_rows) return -1;
    const int64_t tok = token_of_row ? int64_t(token_of_row[row]) : row;
    if (tok < 0) return -1;
    const float m = a.loss_mask[tok];
    const float mp = a.pg_loss_mask ? a.pg_loss_mask[tok] : m;
    return (m == 0.f && mp == 0.f && !a.read_masked_rows) ? -1 : tok;
  };
  auto fetch_token = [&](int64_t row, int64_t tok) {
    ResidentTokenData td{};
    td.tg = -1;
    if (wave0 && tok >= 0) {
      if (tid == 0) {
        td.in = load_token_inputs(a, tok);
        td.tg = targets[tok];
        if (td.tg >= 0 && td.tg < vocab) td.x_target = Row<T>::load1(logits + row * row_stride + td.tg);
        const int32_t sid = sample_ids ? sample_ids[tok] : 0;
        td.den = a.sample_denom ? a.sample_denom[sid] : 1.0f;
        td.pg_den = a.pg_sample_denom ? a.pg_sample_denom[sid] : td.den;
      }
    }
    return td;
  };
  // group g of the resident row into st, following scan_row(): four vectors together while this thread still has
  // four to go, single vectors afterwards (g is a compile-time constant at every call site)
  auto absorb_group = [&](int g, SoftmaxAcc& st, bool& grouped) {
    if (grouped && kU * g + kU - 1 < NV && has(kU * g + kU - 1)) {
      absorb_raw_group<T>(&reg[kU * g < NV - kU ? kU * g : NV - kU], c, st);
    } else {
      grouped = false;
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (kU * g + u < NV && has(kU * g + u)) {
          float v[VN];
          Row<T>::unpack(reg[kU * g + u < NV ? kU * g + u : NV - 1], v);
          scan_absorb(v, c, st);
        }
    }
    // The state is only needed once the whole row is in; without a use here the compiler moves the scan of every
    // group behind the store loop and spills the vectors it was meant to consume on the way.
    asm volatile("" : "+v"(st.m), "+v"(st.s), "+v"(st.t));
    __builtin_amdgcn_sched_barrier(0);  // and one group at a time: hoisting the next group's unpacking spills too
  };
  // writes zeros to the per-token outputs of rows that score a token whose masks are both zero, and zero rows
  auto zero_row = [&](int64_t row) {
    const int64_t t0 = token_of_row ? int64_t(token_of_row[row]) : row;
    if (t0 >= 0 && tid == 0) {
      log_prob[t0] = 0.f;
      entropy[t0] = 0.f;
      lse_out[t0] = 0.f;
      spx_out[t0] = 0.f;
      a.coef_log_prob[t0] = 0.f;
      if (a.coef_entropy) a.coef_entropy[t0] = 0.f;
    }
    u32x4* dv = reinterpret_cast<u32x4*>(dlogits + row * d_stride);
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (has(j)) store_stream(dv + tid + j * THREADS, u32x4{0u, 0u, 0u, 0u});
  };
  // this workgroup's first live row at or after `row` (n_rows or more: none); the dead rows passed on the way are
  // zero-filled here, so the main loop only ever sees live rows
  auto advance = [&](int64_t row) -> int64_t {
    while (row < n_rows && live_token(row) < 0) {
      zero_row(row);
      row += gridDim.x;
    }
    return row;
  };

  // prologue: the first live row is loaded and scanned on its own
  int64_t row = advance(blockIdx.x);
  if (row >= n_rows) return;
  int64_t tok = live_token(row);
  SoftmaxAcc st{kNegHuge, 0.f, 0.f};
  {
    const u32x4* xv = reinterpret_cast<const u32x4*>(logits + row * row_stride);
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (has(j)) reg[j] = load_stream(xv + tid + j * THREADS);
    bool grouped = true;
#pragma unroll
    for (int g = 0; g < kGroups; ++g) absorb_group(g, st, grouped);
  }

  while (true) {
    const int64_t next = advance(row + gridDim.x);
    const bool has_next = next < n_rows;
    const int64_t next_tok = has_next ? live_token(next) : -1;

    // Thread 0's view of the token.  The per-token vectors are a few hundred KB and stay in cache, so fetching them
    // here, behind the merge of the waves' partial states, costs less than carrying them through the scan in
    // registers that every wave would have to set aside.
    const ResidentTokenData td = fetch_token(row, tok);
    TopkGather gathered{};
    TopkRowShape topk_shape{};
    if constexpr (TOPK) {
      if (wave0) {
        int lane = tid;
        asm volatile("" : "+v"(lane));
        gathered = topk_gather<T>(a, logits + row * row_stride, vocab, tok, lane);
        topk_shape = topk_row_shape(a, tok);
      }
    }
    scan_block_merge<THREADS>(st, wave_state);
    if (wave0) {
      float lse = 0.f, spx = 0.f, ent = 0.f, lp = 0.f;
      if (tid == 0) {
        scan_finish(st, td.x_target, td.tg >= 0 && td.tg < vocab, inv_t, lse, spx, ent, lp);
        log_prob[tok] = lp;
        entropy[tok] = ent;
        lse_out[tok] = lse;
        spx_out[tok] = spx;
      }
      // the top-K distillation signal: K gathered logits of this row against the log-sum-exp just found
      float g_topk = 0.f;
      if constexpr (TOPK) {
        int lane = tid;
        asm volatile("" : "+v"(lane));
        g_topk = topk_distill_row(a, gathered, topk_shape, tok, lane_value(lse), inv_t, lane_value(lp),
                                  lane_value(td.in.has_old ? td.in.old_lp : lp), lane_value(td.in.extra_lp), lane,
                                  topk_stage);
      }
      if (tid == 0) {
        relax_amd_policy_loss_args al = a;
        // opaque copies: derived constants (1 + eps, ...) would otherwise be hoisted out of the row loop into vector
        // registers that every wave has to keep for thread 0's sake
        asm volatile("" : "+s"(al.eps_clip), "+s"(al.eps_clip_high), "+s"(al.eps_clip_c), "+s"(al.entropy_coef),
                     "+s"(al.kl_coef), "+s"(al.tis_lo), "+s"(al.tis_hi), "+s"(al.tau_pos), "+s"(al.tau_neg));
        const TokenResult tr = token_terms(al, td.in, lp, ent, false, 0.f, td.den, td.pg_den);
        a.coef_log_prob[tok] = tr.coef_lp;
        if (a.coef_entropy) a.coef_entropy[tok] = tr.coef_ent;
        const float glp = tr.coef_lp * grad_scale, gh = tr.coef_ent * grad_scale;
        const float gsm = TOPK ? glp + g_topk * grad_scale : glp;  // what the row's softmax is subtracted with
        const float b = gh * inv_t;
        bc[0] = -lse * kLog2e;           // k0: p = exp2(x*c + k0)
        bc[1] = -gsm * inv_t + b * spx;  // a0
        bc[2] = -b * inv_t;              // a1: d = p * (a0 + a1*x)
        bc[3] = glp * inv_t;             // added at the target
        bc[4] = (gsm == 0.f && glp == 0.f && gh == 0.f) ? 1.f : 0.f;
        bc_target = td.tg;
      }
    }
    // the barrier's fence also waits for this wave's outstanding loads and stores; all of this row's data is in
    // registers by now, so that costs at most the drain of the previous row's last stores
    __syncthreads();
    const float k0 = bc[0], a0 = bc[1], a1 = bc[2], hot = bc[3];
    const int64_t tg = bc_target;
    const bool emit_zero = bc[4] != 0.f;  // both gradient coefficients vanish: a zero row, whatever the logits hold

    // The row becomes its gradient in place, vector by vector ...
    u32x4* dv = reinterpret_cast<u32x4*>(dlogits + row * d_stride);
    const u32x4* nxv = reinterpret_cast<const u32x4*>(logits + (has_next ? next : row) * row_stride);
    const int tvec = (tg >= 0 && tg < vocab) ? int(tg / VN) : -1;
    const int tsub = int(tg % VN);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));  // recomputed per vector: 19 loop-invariant index registers would not fit
      const int idx = lane_id + j * THREADS;
      float v[VN];
      Row<T>::unpack(reg[j], v);
#pragma unroll
      for (int k = 0; k < VN; ++k) {
        v[k] = fast_exp2(fmaf(v[k], c, k0)) * fmaf(v[k], a1, a0);
        // half a vector in flight at a time: with all eight interleaved the temporaries push parts of the resident
        // row out to scratch (four waves per SIMD cover the latency of the exponentials)
        if (k == VN / 2 - 1) __builtin_amdgcn_sched_barrier(0);
      }
      if (idx == tvec) {  // one lane of the workgroup per row
#pragma unroll
        for (int k = 0; k < VN; ++k)
          if (k == tsub) v[k] += hot;
      }
      reg[j] = emit_zero ? u32x4{0u, 0u, 0u, 0u} : Row<T>::pack(v);
      __builtin_amdgcn_sched_barrier(0);  // one vector at a time: hoisting the next one's unpacking spills
    }
    // ... leaves in one burst of stores, and the next live row arrives in one burst of loads into the same registers
    // (without a next row the row itself is read again: a branch here would cost the precise wait counts, and the
    // last row of a workgroup is one in hundreds)
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));
      if (has(j)) store_stream(dv + lane_id + j * THREADS, reg[j]);
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      int lane_id = tid;
      asm volatile("" : "+v"(lane_id));
      if (has(j)) reg[j] = load_stream(nxv + lane_id + j * THREADS);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!has_next) return;
    // the next row's scan, group by group as its vectors arrive (loads return in the order they were requested)
    st = SoftmaxAcc{kNegHuge, 0.f, 0.f};
    bool grouped = true;
#pragma unroll
    for (int g = 0; g < kGroups; ++g) absorb_group(g, st, grouped);
    row = next;
    tok = next_tok;
  }
}

#define RELAX_AMD_RESIDENT(NVF, PARTIAL)                                                                             \
  if (full == NVF && partial == PARTIAL) {                                                                            \
    if (a.topk_ids)                                                                                                   \
      hipLaunchKernelGGL((actor_step_resident_kernel<T, NVF, PARTIAL, true>), grid, block, 0, stream, logits,        \
                         row_stride, vocab, n_rows, token_of_row, sample_ids, targets, inv_t * kLog2e, inv_t, a,     \
                         grad_scale, log_prob, entropy, lse, spx, dlogits, d_stride);                                \
    else                                                                                                              \
      hipLaunchKernelGGL((actor_step_resident_kernel<T, NVF, PARTIAL, false>), grid, block, 0, stream, logits,       \
                         row_stride, vocab, n_rows, token_of_row, sample_ids, targets, inv_t * kLog2e, inv_t, a,     \
                         grad_scale, log_prob, entropy, lse, spx, dlogits, d_stride);                                \
    return check_launch("actor_step_resident");                                                                      \
  }

template <typename T>
int launch_actor_step_resident(const T* logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
                               const int32_t* token_of_row, const int32_t* sample_ids, const int64_t* targets,
                               float inv_t, const relax_amd_policy_loss_args& a, float grad_scale, float* log_prob,
                               float* entropy, float* lse, float* spx, T* dlogits, int64_t d_stride,
                               int compute_units, hipStream_t stream) {
  constexpr int VN = Row<T>::kPerVec, THREADS = resident_threads<T>();
  // the workgroup must be as wide as the forward-only kernel's for this row length: both scan in the same order
  if (vocab % VN != 0 || scan_threads(vocab, VN) != THREADS) return RELAX_AMD_EUNSUPPORTED;
  const int64_t nvec = vocab / VN;
  const int full = int(nvec / THREADS);
  const bool partial = nvec % THREADS != 0;
  const int64_t slots = int64_t(compute_units) * (1024 / THREADS);  // persistent workgroups: as many as fit the chip
  const dim3 grid(static_cast<unsigned>(n_rows < slots ? n_rows : slots)), block(THREADS);
  if constexpr (sizeof(T) == 2) {
    // vocabularies of 163840 (20480 vectors) and up to it, 151936 / 152064 (18992 / 19008), 128256 / 129280
    // (16032 / 16160), 131072 (16384),
    // 100352 / 102400 (12544 / 12800) entries
    RELAX_AMD_RESIDENT(20, false)
    RELAX_AMD_RESIDENT(19, true)
    RELAX_AMD_RESIDENT(18, true)
    RELAX_AMD_RESIDENT(15, true)
    RELAX_AMD_RESIDENT(16, false)
    RELAX_AMD_RESIDENT(12, true)
    // and the short end of the 1024-thread rows: 65536 entries (8192 vectors) and 57352 .. 65528 (64000: 8000)
    RELAX_AMD_RESIDENT(8, false)
    RELAX_AMD_RESIDENT(7, true)
  } else {
    // fp32 rows of 32000 entries (8000 vectors: 7 per thread and 832 lanes with an eighth), of 32768, of
    // 49156 .. 53248 (50304: 12576 vectors), of 61444 .. 65532 (64000) and of 65536
    RELAX_AMD_RESIDENT(7, true)
    RELAX_AMD_RESIDENT(8, false)
    RELAX_AMD_RESIDENT(12, true)
    RELAX_AMD_RESIDENT(15, true)
    RELAX_AMD_RESIDENT(16, false)
  }
  return RELAX_AMD_EUNSUPPORTED;
}
#undef RELAX_AMD_RESIDENT

template int launch_actor_step_resident<float>(const float*, int64_t, int64_t, int64_t, const int32_t*, const int32_t*,
                                               const int64_t*, float, const relax_amd_policy_loss_args&, float, float*,
                                               float*, float*, float*, float*, int64_t, int, hipStream_t);
template int launch_actor_step_resident<bf16_t>(const bf16_t*, int64_t, int64_t, int64_t, const int32_t*,
                                                const int32_t*, const int64_t*, float,
                                                const relax_amd_policy_loss_args&, float, float*, float*, float*,
                                                float*, bf16_t*, int64_t, int, hipStream_t);
template int launch_actor_step_resident<f16_t>(const f16_t*, int64_t, int64_t, int64_t, const int32_t*, const int32_t*,
                                               const int64_t*, float, const relax_amd_policy_loss_args&, float, float*,
                                               float*, float*, float*, f16_t*, int64_t, int, hipStream_t);

}  // namespace relax_amd
