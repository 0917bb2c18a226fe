// Fused actor step with every row shared between eight one-shot workgroups: the same computation and the same bits
// as actor_step_resident_kernel (log-prob + entropy forward, per-token policy-loss coefficients, dlogits backward, each
// logit read once and each gradient written once), in the launch shape this memory system streams fastest: many small
// workgroups that touch their memory once and retire, dispatched in address order (a mixed read / write stream of
// this shape moves 6.1 - 6.6 TB/s on the box where 256 persistent row-sized streams move 5.6; this kernel on the
// 65536 x 151936 bf16 step: 5.64 - 5.74 ms compiled for three waves per SIMD, 5.74 - 5.89 for four, where the
// persistent kernel takes 6.44 - 6.58; 6.0 ms with 256-thread and 6.3 ms with 64-thread workgroups).
//
// A row is scanned by 1024 "virtual threads" exactly as scan_row() lays it out for a 1024-thread workgroup (virtual
// thread t takes the 16-byte vectors t, t + 1024, ...; four at a time while it has four to go, then single ones).  A
// workgroup here is 128 of those virtual threads (two waves: virtual waves 2q and 2q + 1 of the row), holds its
// share of the row in registers (19 vectors per thread at V = 151936 bf16), reduces each wave to its (max, sum exp,
// sum exp * x) triple by the same butterfly, publishes the two triples, fetches the row's sixteen, merges them in
// wave order as scan_block_merge() does, and turns its registers into the gradient.  Log-probs, entropy and gradients
// are therefore bit-identical to the forward-only kernel's and the other fused kernels'.
//
// Exchange: the tagged ring of row_exchange.h, a slot of 16 x 3 words per row; a workgroup that gives up its wait
// writes NaN log-probs instead of hanging.
//
// Rows whose share does not fit the registers of three waves per SIMD (16-bit rows of more than 20 vectors per thread,
// fp32 rows of more than 16: vocabularies of 100352 .. 163840 entries as fp32, 200 k .. 262 k entries as 16-bit,
// 248320 as either) keep twelve to nineteen vectors of every thread's share in LDS, put there by global -> LDS loads
// without a register in between (LDS_VECS).  An fp32 row of 151936 entries is thereby read once as it is (5.85 -
// 5.95 ms per 32768 rows whether its values are widened bf16 or genuinely fp32).
//
// Replaces, like the other fused kernels, _VocabParallelLogProbEntropy.forward + .backward
// (relax/utils/training/ppo_utils.py:481-629) and the per-token part of policy_loss_function
// (relax/backends/megatron/loss.py:961-1100) for one micro-batch.
//
// As in actor_step_resident.hip the row sits at the edge of the register file:
// hipcc-flags: -mllvm -amdgpu-use-amdgpu-trackers=1
#include <atomic>

#include "actor_step_resident.h"
#include "device_utils.h"
#include "loss_math.h"
#include "opd_topk_math.h"
#include "row_exchange.h"
#include "row_scan.h"

namespace relax_amd {

constexpr int kRowWaves = 16;             // waves of the 1024 virtual threads of a row
constexpr int kSlotWords = kRowWaves * 3;
constexpr int kSplitThreads = 128;        // virtual threads per workgroup
constexpr int kSplit = 1024 / kSplitThreads;
constexpr size_t kRingWords = size_t(kRing) * kSlotWords;

// the exchange ring and its status words
static __device__ __align__(256) unsigned long long split_ring[kRingWords + kRingTailWords];
// The logits at a token's top-K ids, gathered once per row: each workgroup of a row fetches its share of the K
// scattered entries and publishes them here (one tagged word per entry, the ring's tags and status words), every
// workgroup's first wave collects all K.  Gathered by each of the eight workgroups for itself, the K scattered lines
// crossed the fabric eight times per row (3.4 GB on 65536 x 151936 rows with K = 64, a tenth of the step's traffic).
constexpr size_t kTopkRingWords = size_t(kRing) * RELAX_AMD_FUSED_TOPK_MAX;
static __device__ __align__(256) unsigned long long split_topk_ring[kTopkRingWords];

// scan_absorb() over the values of kScanUnroll raw vectors (as in actor_step_resident.hip: same arithmetic, same
// order)
// KEEP: whether the second walk may use the values the first one unpacked (32 registers for 16-bit rows); without, the
// raw vectors are marked as changed in between, so that the compiler unpacks them again
template <typename T, bool KEEP = true>
__device__ __forceinline__ void split_absorb_raw_group(u32x4* raw, float c, SoftmaxAcc& st) {
  constexpr int VN = Row<T>::kPerVec;
  float vmax = 0.f;
#pragma unroll
  for (int u = 0; u < kScanUnroll; ++u) {
    float v[VN];
    Row<T>::unpack(raw[u], v);
#pragma unroll
    for (int k = 0; k < VN; ++k) vmax = (u == 0 && k == 0) ? v[0] : fmaxf(vmax, v[k]);
    __builtin_amdgcn_sched_barrier(0);
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
    if constexpr (!KEEP) asm volatile("" : "+v"(raw[u].x), "+v"(raw[u].y), "+v"(raw[u].z), "+v"(raw[u].w));
    float v[VN];
    Row<T>::unpack(raw[u], v);  // the compiler keeps the first walk's values: with wave 0's share parked in LDS
                                // during thread 0's arithmetic there is room for them next to the row
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      const float e = fast_exp2(fmaf(v[k], c, -st.m));
      st.s = __fadd_rn(st.s, e);
      st.t = fmaf(e, v[k], st.t);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// Lane 0's triple of this wave (the butterfly's merge is not symmetric in its last bits: scan_block_merge() takes lane
// 0's) into the row's slot, as three tagged words written by lanes 0..2.
__device__ __forceinline__ void split_publish(unsigned long long* slot, unsigned tag, int vt, const SoftmaxAcc& st) {
  const float m0 = lane_value(st.m), s0 = lane_value(st.s), t0 = lane_value(st.t);
  const int lane = vt & (kWave - 1), vwave = vt / kWave;
  if (lane < 3) {
    const float val = lane == 0 ? m0 : (lane == 1 ? s0 : t0);
    exchange_store(slot + vwave * 3 + lane, tag, val);
  }
}

// Wave 0 of a workgroup: lanes 0 .. 3 * ROW_WAVES - 1 fetch one word of the row's triples each (waiting, boundedly,
// for the tag of this launch and lap), then every lane merges the ROW_WAVES triples in wave order, as thread 0 of a
// workgroup of that many waves does in scan_block_merge().
template <int ROW_WAVES = kRowWaves>
__device__ __forceinline__ SoftmaxAcc split_collect(const unsigned long long* slot, unsigned tag, int tid,
                                                    unsigned max_polls, unsigned* status, bool& any_gave_up) {
  float word = 0.f;
  bool gave_up = false;
  if (tid < ROW_WAVES * 3) gave_up = !exchange_wait(slot + tid, tag, max_polls, status, word);
  any_gave_up = __any(gave_up);
  if (any_gave_up && tid == 0) exchange_report_give_up(status);
  auto of_lane = [&](int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(word), l)); };
  SoftmaxAcc whole{of_lane(0), of_lane(1), of_lane(2)};
#pragma unroll
  for (int i = 1; i < ROW_WAVES; ++i) scan_merge(whole, of_lane(3 * i), of_lane(3 * i + 1), of_lane(3 * i + 2));
  return whole;
}

// this workgroup's LDS_VECS x 128 vectors of the row that live in LDS (only instantiated, and only allocated, for
// LDS_VECS > 0)
template <int LDS_VECS>
__device__ __forceinline__ u32x4* split_lds_rows() {
  __shared__ u32x4 rows[LDS_VECS * kSplitThreads];
  return rows;
}

// where wave 0's share waits during thread 0's serial stretch (only instantiated, and only allocated, for PARK > 0)
template <int PARK>
__device__ __forceinline__ u32x4 (*split_parked())[kWave] {
  __shared__ u32x4 parked[PARK][kWave];
  return parked;
}

// ROW_THREADS: the virtual threads that scan a row, i.e. the width scan_threads() gives the forward-only kernel for this
// row length (1024, or 512 for rows of 2048 .. 7167 vectors); ROW_THREADS / 128 workgroups share a row.
// WAVES_MIN / WAVES_MAX: the waves per SIMD the register allocation aims for (see split_waves_min()).
// LDS_VECS: rows longer than the register file holds at three waves per SIMD (16-bit vocabularies above 163840 entries)
// keep the first LDS_VECS vectors of every thread's share in LDS, where global -> LDS loads put them without a
// register in between; wave 0 then has registers to spare for thread 0's serial stretch and parks nothing.
template <typename T, int NVF, bool PARTIAL, bool TOPK, int ROW_THREADS, int WAVES_MIN, int WAVES_MAX, int LDS_VECS = 0>
__global__ __launch_bounds__(kSplitThreads) __attribute__((amdgpu_waves_per_eu(WAVES_MIN, WAVES_MAX)))
void actor_step_split_kernel(
    const T* __restrict__ logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
    const int32_t* __restrict__ token_of_row, const int32_t* __restrict__ sample_ids,
    const int64_t* __restrict__ targets, float c, float inv_t, relax_amd_policy_loss_args a, float grad_scale,
    float* __restrict__ log_prob, float* __restrict__ entropy, float* __restrict__ lse_out,
    float* __restrict__ spx_out, T* __restrict__ dlogits, int64_t d_stride, unsigned long long* __restrict__ ring,
    unsigned long long* __restrict__ topk_ring, unsigned laps, unsigned max_polls, unsigned wait_tag_offset) {
  constexpr int kU = kScanUnroll, kParts = ROW_THREADS / kSplitThreads;
  constexpr int VN = Row<T>::kPerVec;
  constexpr int NV = NVF + (PARTIAL ? 1 : 0);
  constexpr int kGroups = (NV + kU - 1) / kU;
  __shared__ float bc[5];
  __shared__ int64_t bc_target;
  __shared__ float topk_stage[TOPK ? kTopkStageFloats : 1];
  // vectors of wave 0's share that wait in LDS during thread 0's serial stretch (see there): all of them, or as many
  // as leave room for eight workgroups per CU next to the top-K term's staging area
  constexpr int kPark = LDS_VECS > 0 ? 0 : (NV < (TOPK ? 15 : 19) ? NV : (TOPK ? 15 : 19));
  u32x4(*parked)[kWave] = nullptr;
  if constexpr (kPark > 0) parked = split_parked<kPark>();
  constexpr int NR = NV - LDS_VECS;  // vectors of the share in registers
  static_assert(LDS_VECS <= NVF && NR >= kU, "only full vector positions go to LDS");
  const int tid = threadIdx.x;
  const bool wave0 = __builtin_amdgcn_readfirstlane(tid) < kWave;
  const unsigned part = blockIdx.x % kParts;
  const int64_t row = blockIdx.x / kParts;
  const int vt = int(part) * kSplitThreads + tid;  // virtual thread of the row
  const int rem = int(vocab / VN) - NVF * ROW_THREADS;
  auto has = [&](int j) -> bool { return j < NVF || (PARTIAL && j == NVF && vt < rem); };
  u32x4* dv = reinterpret_cast<u32x4*>(dlogits + row * d_stride);

  // token of the row, or -1 when the row scores nothing or both of its masks are zero (uniform over the workgroup)
  int64_t tok = token_of_row ? int64_t(token_of_row[row]) : row;
  const int64_t t0 = tok;
  if (tok >= 0) {
    const float m = a.loss_mask[tok];
    const float mp = a.pg_loss_mask ? a.pg_loss_mask[tok] : m;
    if (m == 0.f && mp == 0.f && !a.read_masked_rows) tok = -1;
  }
  if (tok < 0) {  // a zero row: no read, no exchange
    if (t0 >= 0 && part == 0 && tid == 0) {
      log_prob[t0] = 0.f;
      entropy[t0] = 0.f;
      lse_out[t0] = 0.f;
      spx_out[t0] = 0.f;
      a.coef_log_prob[t0] = 0.f;
      if (a.coef_entropy) a.coef_entropy[t0] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (has(j)) store_stream(dv + vt + j * ROW_THREADS, u32x4{0u, 0u, 0u, 0u});
    return;
  }

  const u32x4* xv = reinterpret_cast<const u32x4*>(logits + row * row_stride);
  // this workgroup's share of the row's K gathered logits: entries part * chunk .. + chunk, one per lane of the second
  // wave; the id is requested ahead of the row, the logit behind it
  int my_k = -1;
  int64_t my_id = -1;
  if constexpr (TOPK) {
    const int kmax = a.topk_k, chunk = (kmax + kParts - 1) / kParts, t1 = tid - kWave;
    if (t1 >= 0 && t1 < chunk && int(part) * chunk + t1 < kmax) {
      my_k = int(part) * chunk + t1;
      my_id = a.topk_ids[tok * kmax + my_k];
    }
  }
  u32x4 reg[NR];
  if constexpr (LDS_VECS > 0) {
    u32x4* rows = split_lds_rows<LDS_VECS>();
    const int wave_base = __builtin_amdgcn_readfirstlane(tid / kWave) * kWave;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      if (j < LDS_VECS)
        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(xv + vt + j * ROW_THREADS),
                                         (__attribute__((address_space(3))) void*)(rows + j * kSplitThreads + wave_base),
                                         16, 0, 0);
      else if (has(j))
        reg[j - LDS_VECS] = load_stream(xv + vt + j * ROW_THREADS);
    }
  } else {
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (has(j)) reg[j] = load_stream(xv + vt + j * ROW_THREADS);
  }
  // vector j of this thread's share
  auto vec = [&](int j) -> u32x4 {
    if constexpr (LDS_VECS > 0) {
      if (j < LDS_VECS) return split_lds_rows<LDS_VECS>()[(j < LDS_VECS ? j : 0) * kSplitThreads + tid];
    }
    return reg[j < LDS_VECS ? 0 : j - LDS_VECS];
  };
  // this launch's tags: the counter was advanced by `laps` in front of the launch
  const unsigned tag = exchange_tag(reinterpret_cast<const unsigned*>(ring + kRingWords), laps, row);
  float my_gathered = 0.f;
  if constexpr (TOPK) {
    if (my_k >= 0) my_gathered = topk_gather_one<T>(a, logits + row * row_stride, vocab, my_id);
  }

  // the scan, group by group as the vectors arrive, in scan_row()'s order
  SoftmaxAcc st{kNegHuge, 0.f, 0.f};
  bool grouped = true;
#pragma unroll
  for (int g = 0; g < kGroups; ++g) {
    if (grouped && kU * g + kU - 1 < NV && has(kU * g + kU - 1)) {
      if constexpr (LDS_VECS > 0) {
        u32x4 grp[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) grp[u] = vec((kU * g < NV - kU ? kU * g : NV - kU) + u);
        split_absorb_raw_group<T, false>(grp, c, st);
      } else {
        split_absorb_raw_group<T>(&reg[kU * g < NV - kU ? kU * g : NV - kU], c, st);
      }
    } else {
      grouped = false;
#pragma unroll
      for (int u = 0; u < kU; ++u)
        if (kU * g + u < NV && has(kU * g + u)) {
          float v[VN];
          Row<T>::unpack(vec(kU * g + u < NV ? kU * g + u : NV - 1), v);
          scan_absorb(v, c, st);
        }
    }
    asm volatile("" : "+v"(st.m), "+v"(st.s), "+v"(st.t));
    __builtin_amdgcn_sched_barrier(0);
  }
  // each wave to its triple (scan_block_merge()'s first half), published by its lanes 0..2
  wave_butterfly([&](auto o) {
    constexpr int O = decltype(o)::value;
    scan_merge(st, lane_xor<O>(st.m), lane_xor<O>(st.s), lane_xor<O>(st.t));
  });
  unsigned long long* slot = ring + size_t(row % kRing) * kSlotWords;
  split_publish(slot, tag, vt, st);
  unsigned long long* topk_slot = nullptr;
  if constexpr (TOPK) {
    topk_slot = topk_ring + size_t(row % kRing) * RELAX_AMD_FUSED_TOPK_MAX;
    if (my_k >= 0) exchange_store(topk_slot + my_k, tag, my_gathered);
  }

  if (wave0) {
    // thread 0 runs a serial stretch from here to the barrier while the other waves of the workgroup wait
    __builtin_amdgcn_s_setprio(3);
    // wave 0's share of the row waits in LDS meanwhile: thread 0's loss arithmetic needs some thirty registers of its
    // own, which every wave of the kernel would otherwise have to set aside next to the row
#pragma unroll
    for (int j = 0; j < kPark; ++j) parked[j][tid] = reg[j];
    // thread 0's view of the token, fetched while the triples travel
    TokenInputs tin{};
    float x_target = 0.f, den = 1.f, pg_den = 1.f;
    int64_t tg = -1;
    if (tid == 0) {
      tin = load_token_inputs(a, tok);
      tg = targets[tok];
      if (tg >= 0 && tg < vocab) x_target = Row<T>::load1(logits + row * row_stride + tg);
      const int32_t sid = sample_ids ? sample_ids[tok] : 0;
      den = a.sample_denom ? a.sample_denom[sid] : 1.0f;
      pg_den = a.pg_sample_denom ? a.pg_sample_denom[sid] : den;
    }
    TopkGather gathered{};
    TopkRowShape topk_shape{};
    if constexpr (TOPK) {
      int lane = tid;
      asm volatile("" : "+v"(lane));
      gathered = topk_gather_meta(a, tok, lane);
      topk_shape = topk_row_shape(a, tok);
    }
    bool any_gave_up = false;
    const SoftmaxAcc whole = split_collect<ROW_THREADS / kWave>(slot, tag + wait_tag_offset, tid, max_polls,
                                                                reinterpret_cast<unsigned*>(ring + kRingWords), any_gave_up);
    if constexpr (TOPK) {
      // the row's gathered logits, entry lane + 64 i from the workgroup that fetched it
      unsigned* status = reinterpret_cast<unsigned*>(ring + kRingWords);
      bool gave_up = any_gave_up;
#pragma unroll
      for (int i = 0; i < kTopkPerLane; ++i) {
        const int k = tid + i * kWave;
        if (k < a.topk_k && !gave_up)
          gave_up = !exchange_wait(topk_slot + k, tag + wait_tag_offset, max_polls, status, gathered.x[i]);
      }
      const bool any_topk_gave_up = __any(gave_up);
      if (any_topk_gave_up && !any_gave_up && tid == 0) exchange_report_give_up(status);
      any_gave_up = any_topk_gave_up;
    }
    float lse = 0.f, spx = 0.f, ent = 0.f, lp = 0.f;
    if (tid == 0) {
      scan_finish(whole, x_target, tg >= 0 && tg < vocab, inv_t, lse, spx, ent, lp);
      if (any_gave_up) lp = lse = __builtin_nanf("");
      if (part == 0) {
        log_prob[tok] = lp;
        entropy[tok] = ent;
        lse_out[tok] = lse;
        spx_out[tok] = spx;
      }
    }
    float g_topk = 0.f;
    if constexpr (TOPK) {
      int lane = tid;
      asm volatile("" : "+v"(lane));
      g_topk = topk_distill_row(a, gathered, topk_shape, tok, lane_value(lse), inv_t, lane_value(lp),
                                lane_value(tin.has_old ? tin.old_lp : lp), lane_value(tin.extra_lp), lane, topk_stage,
                                part == 0);
    }
    if (tid == 0) {
      relax_amd_policy_loss_args al = a;
      asm volatile("" : "+s"(al.eps_clip), "+s"(al.eps_clip_high), "+s"(al.eps_clip_c), "+s"(al.entropy_coef),
                   "+s"(al.kl_coef), "+s"(al.tis_lo), "+s"(al.tis_hi), "+s"(al.tau_pos), "+s"(al.tau_neg));
      const TokenResult tr = token_terms(al, tin, lp, ent, false, 0.f, den, pg_den);
      if (part == 0) {
        a.coef_log_prob[tok] = tr.coef_lp;
        if (a.coef_entropy) a.coef_entropy[tok] = tr.coef_ent;
      }
      const float glp = tr.coef_lp * grad_scale, gh = tr.coef_ent * grad_scale;
      const float gsm = TOPK ? glp + g_topk * grad_scale : glp;
      const float b = gh * inv_t;
      bc[0] = -lse * kLog2e;           // k0: p = exp2(x*c + k0)
      bc[1] = -gsm * inv_t + b * spx;  // a0
      bc[2] = -b * inv_t;              // a1: d = p * (a0 + a1*x)
      bc[3] = glp * inv_t;             // added at the target
      bc[4] = (gsm == 0.f && glp == 0.f && gh == 0.f) ? 1.f : 0.f;
      bc_target = tg;
    }
#pragma unroll
    for (int j = 0; j < kPark; ++j) reg[j] = parked[j][tid];
    __builtin_amdgcn_s_setprio(0);
  }
  __syncthreads();
  const float k0 = bc[0], a0 = bc[1], a1 = bc[2], hot = bc[3];
  const int64_t tgt = bc_target;
  const bool emit_zero = bc[4] != 0.f;
  const int tvec = (tgt >= 0 && tgt < vocab) ? int(tgt / VN) : -1;
  const int tsub = int(tgt % VN);
  if (emit_zero) {  // uniform over the workgroup: both gradient coefficients vanish, a zero row whatever the logits hold
#pragma unroll
    for (int j = 0; j < NV; ++j)
      if (has(j)) store_stream(dv + vt + j * ROW_THREADS, u32x4{0u, 0u, 0u, 0u});
    return;
  }
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    int lane_id = vt;
    asm volatile("" : "+v"(lane_id));
    const int idx = lane_id + j * ROW_THREADS;
    float v[VN];
    Row<T>::unpack(vec(j), v);
#pragma unroll
    for (int k = 0; k < VN; ++k) {
      v[k] = fast_exp2(fmaf(v[k], c, k0)) * fmaf(v[k], a1, a0);
      if (k == VN / 2 - 1) __builtin_amdgcn_sched_barrier(0);
    }
    u32x4 out = Row<T>::pack(v);
    // The element at the target gets `hot` added before it is rounded.  One wave in 300 holds it: that wave takes a
    // jump (the ballot is wave-uniform) and packs the vector again; as a per-lane select on every vector the same
    // update costs two vector instructions per element, an eighth of the kernel's arithmetic.
    if (__builtin_amdgcn_ballot_w64(idx == tvec) != 0ull) {
#pragma unroll
      for (int k = 0; k < VN; ++k)
        if (idx == tvec && k == tsub) v[k] += hot;
      out = Row<T>::pack(v);
    }
    if (has(j)) store_stream(dv + idx, out);
    __builtin_amdgcn_sched_barrier(0);
  }
}

namespace {
ExchangeRingCache ring_cache, topk_ring_cache;
// relax_amd_set_exchange_wait: the bound of a workgroup's wait and an offset added to the tag it waits for
std::atomic<unsigned> g_max_polls{kWaitPolls}, g_wait_tag_offset{0u};
}  // namespace

unsigned exchange_max_polls() { return g_max_polls.load(std::memory_order_relaxed); }
unsigned exchange_wait_tag_offset() { return g_wait_tag_offset.load(std::memory_order_relaxed); }

static int split_ring_of_device(unsigned long long** ring) {
  return exchange_ring_of_device(ring_cache, reinterpret_cast<const void*>(&split_ring), "actor_step_split", ring);
}
static int split_topk_ring_of_device(unsigned long long** ring) {
  return exchange_ring_of_device(topk_ring_cache, reinterpret_cast<const void*>(&split_topk_ring), "actor_step_split",
                                 ring);
}

// Waves per SIMD the kernel is compiled for.  Long 16-bit rows without the top-K term run fastest with three (six
// workgroups per CU, up to 168 registers a lane: 5.64 - 5.66 ms on the 65536 x 151936 step where four give 5.74 and
// two 6.03; rows of 15 and more vectors per thread all gain 1 - 2.5 %), the top-K instantiations and rows of up to 13
// vectors per thread with four or more (their thread 0 works longer per row, or they need few registers anyway).
template <int NV, bool TOPK, int VN>
constexpr int split_waves_min() {
  return (!TOPK && VN == 8 && NV >= 15) ? 3 : 4;
}
template <int NV, bool TOPK, int VN>
constexpr int split_waves_max() {
  return (!TOPK && VN == 8 && NV >= 15) ? 3 : 8;
}
#define RELAX_AMD_SPLIT_KERNEL(WIDTH, NVF, PARTIAL, TOPK)                                                             \
  actor_step_split_kernel<T, NVF, PARTIAL, TOPK, WIDTH, split_waves_min<NVF + (PARTIAL ? 1 : 0), TOPK, VN>(),         \
                          split_waves_max<NVF + (PARTIAL ? 1 : 0), TOPK, VN>()>
#define RELAX_AMD_SPLIT_ROW(WIDTH, NVF, PARTIAL)                                                                      \
  if (width == WIDTH && full == NVF && partial == PARTIAL) {                                                          \
    if (a.topk_ids)                                                                                                   \
      hipLaunchKernelGGL((RELAX_AMD_SPLIT_KERNEL(WIDTH, NVF, PARTIAL, true)), grid, block, 0, stream, logits,        \
                         row_stride, vocab, n_rows, token_of_row, sample_ids, targets, inv_t * kLog2e, inv_t, a,     \
                         grad_scale, log_prob, entropy, lse, spx, dlogits, d_stride, ring, topk_ring, laps,          \
                         max_polls, tag_offset);                                                                      \
    else                                                                                                              \
      hipLaunchKernelGGL((RELAX_AMD_SPLIT_KERNEL(WIDTH, NVF, PARTIAL, false)), grid, block, 0, stream, logits,       \
                         row_stride, vocab, n_rows, token_of_row, sample_ids, targets, inv_t * kLog2e, inv_t, a,     \
                         grad_scale, log_prob, entropy, lse, spx, dlogits, d_stride, ring, topk_ring, laps,          \
                         max_polls, tag_offset);                                                                      \
    return check_launch("actor_step_split");                                                                          \
  }
#define RELAX_AMD_SPLIT(NVF, PARTIAL) RELAX_AMD_SPLIT_ROW(1024, NVF, PARTIAL)
// Rows of more vectors per thread than the register file holds at three waves per SIMD (16-bit rows of more than 20,
// fp32 rows of more than 16): part of every thread's share sits in LDS.  16-bit: twelve or thirteen vectors (24 - 26 KB
// of the 26.7 a workgroup can have when six share a CU), three waves per SIMD.  fp32 rows of up to 40 vectors per
// thread (100352 .. 163840 entries): thirteen in LDS, three waves; of 61 (248320 entries): nineteen in LDS (38 KB), two
// waves.  With the top-K term (4 KB of LDS more, a longer serial stretch): sixteen in LDS and two waves per SIMD.
template <int NV, bool TOPK, int VN>
constexpr int split_lds_vecs() {
  return TOPK ? 16 : (VN == 4 && NV > 40) ? 19 : (VN == 8 && NV <= 25) ? 12 : 13;
}
template <int NV, bool TOPK, int VN>
constexpr int split_lds_waves() {
  return (TOPK || (VN == 4 && NV > 40)) ? 2 : 3;
}
#define RELAX_AMD_SPLIT_LDS_KERNEL(NVF, PARTIAL, TOPK)                                                                \
  actor_step_split_kernel<T, NVF, PARTIAL, TOPK, 1024, split_lds_waves<NVF + (PARTIAL ? 1 : 0), TOPK, VN>(),          \
                          split_lds_waves<NVF + (PARTIAL ? 1 : 0), TOPK, VN>(),                                       \
                          split_lds_vecs<NVF + (PARTIAL ? 1 : 0), TOPK, VN>()>
#define RELAX_AMD_SPLIT_LDS(NVF, PARTIAL, WITH_TOPK)                                                                  \
  if (width == 1024 && full == NVF && partial == PARTIAL) {                                                           \
    if (a.topk_ids) {                                                                                                 \
      if constexpr (WITH_TOPK)                                                                                        \
        hipLaunchKernelGGL((RELAX_AMD_SPLIT_LDS_KERNEL(NVF, PARTIAL, true)), grid, block, 0, stream, logits,         \
                           row_stride, vocab, n_rows, token_of_row, sample_ids, targets, inv_t * kLog2e, inv_t, a,   \
                           grad_scale, log_prob, entropy, lse, spx, dlogits, d_stride, ring, topk_ring, laps,        \
                           max_polls, tag_offset);                                                                    \
    } else {                                                                                                          \
      hipLaunchKernelGGL((RELAX_AMD_SPLIT_LDS_KERNEL(NVF, PARTIAL, false)), grid, block, 0, stream, logits,          \
                         row_stride, vocab, n_rows, token_of_row, sample_ids, targets, inv_t * kLog2e, inv_t, a,     \
                         grad_scale, log_prob, entropy, lse, spx, dlogits, d_stride, ring, topk_ring, laps,          \
                         max_polls, tag_offset);                                                                      \
    }                                                                                                                 \
    return check_launch("actor_step_split");                                                                          \
  }

template <typename T>
int launch_actor_step_split(const T* logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
                            const int32_t* token_of_row, const int32_t* sample_ids, const int64_t* targets,
                            float inv_t, const relax_amd_policy_loss_args& a, float grad_scale, float* log_prob,
                            float* entropy, float* lse, float* spx, T* dlogits, int64_t d_stride,
                            hipStream_t stream) {
  constexpr int VN = Row<T>::kPerVec;
  const int width = scan_threads(vocab, VN);  // the virtual threads of a row: the forward-only kernel's workgroup
  if (vocab % VN != 0 || width < 512 || n_rows * kSplit > 2147483647LL) return RELAX_AMD_EUNSUPPORTED;
  const int64_t nvec = vocab / VN;
  const int full = int(nvec / width);
  const bool partial = nvec % width != 0;
  // the row shapes launch_actor_step_resident is built for, and 16-bit rows of 3585 .. 4096 and 6145 .. 6656 vectors
  // (32000 / 32768 and 50304 entries) scanned by 512 virtual threads
  if (width == 512) {
    if (sizeof(T) != 2 || !((full == 7 && partial) || (full == 8 && !partial) || (full == 12 && partial)))
      return RELAX_AMD_EUNSUPPORTED;
  } else if constexpr (sizeof(T) == 2) {
    const bool lds_row = (full == 24 && partial) || (full == 30 && partial) || (full == 31 && partial) ||
                         (full == 32 && !partial);
    if (!(lds_row || (full == 20 && !partial) || (full == 19 && partial) || (full == 18 && partial) ||
          (full == 15 && partial) || (full == 16 && !partial) || (full == 12 && partial) || (full == 8 && !partial) ||
          (full == 7 && partial)))
      return RELAX_AMD_EUNSUPPORTED;
  } else {
    // fp32: 100352 / 102400 (25088 / 25600 vectors), 128256 / 129280 (32064 / 32320), 131072 (32768), 151936 / 152064 /
    // 154880 (37984 / 38016 / 38720), 163840 (40960), 248320 (62080; the top-K term is left to the two-walk kernel)
    const bool lds_row = (full == 24 && partial) || (full == 25 && !partial) || (full == 31 && partial) ||
                         (full == 32 && !partial) || (full == 37 && partial) || (full == 40 && !partial) ||
                         (full == 60 && partial);
    if (full == 60 && a.topk_ids) return RELAX_AMD_EUNSUPPORTED;
    if (!(lds_row || (full == 7 && partial) || (full == 8 && !partial) || (full == 12 && partial) ||
          (full == 15 && partial) || (full == 16 && !partial)))
      return RELAX_AMD_EUNSUPPORTED;
  }
  unsigned long long* ring = nullptr;
  if (int rc = split_ring_of_device(&ring)) return rc;
  unsigned long long* topk_ring = nullptr;
  if (int rc = split_topk_ring_of_device(&topk_ring)) return rc;
  const unsigned laps = unsigned((n_rows + kRing - 1) / kRing);
  const unsigned max_polls = exchange_max_polls();
  const unsigned tag_offset = exchange_wait_tag_offset();
  hipLaunchKernelGGL(exchange_ring_advance_kernel<kRingWords>, dim3(1), dim3(256), 0, stream, ring, laps,
                     topk_ring, kTopkRingWords);
  const dim3 grid(static_cast<unsigned>(n_rows * (width / kSplitThreads))), block(kSplitThreads);
  if constexpr (sizeof(T) == 2) {
    RELAX_AMD_SPLIT_ROW(512, 7, true)
    RELAX_AMD_SPLIT_ROW(512, 8, false)
    RELAX_AMD_SPLIT_ROW(512, 12, true)
    // 200064 / 201088 / 202048 (25008 / 25136 / 25256 vectors), 250880 (31360), 256000 (32000), 262144 (32768) entries
    RELAX_AMD_SPLIT_LDS(24, true, true)
    RELAX_AMD_SPLIT_LDS(30, true, true)
    RELAX_AMD_SPLIT_LDS(31, true, true)
    RELAX_AMD_SPLIT_LDS(32, false, true)
    RELAX_AMD_SPLIT(20, false)
    RELAX_AMD_SPLIT(19, true)
    RELAX_AMD_SPLIT(18, true)
    RELAX_AMD_SPLIT(15, true)
    RELAX_AMD_SPLIT(16, false)
    RELAX_AMD_SPLIT(12, true)
    RELAX_AMD_SPLIT(8, false)
    RELAX_AMD_SPLIT(7, true)
  } else {
    RELAX_AMD_SPLIT_LDS(37, true, true)
    RELAX_AMD_SPLIT_LDS(31, true, true)
    RELAX_AMD_SPLIT_LDS(32, false, true)
    RELAX_AMD_SPLIT_LDS(40, false, true)
    RELAX_AMD_SPLIT_LDS(24, true, true)
    RELAX_AMD_SPLIT_LDS(25, false, true)
    RELAX_AMD_SPLIT_LDS(60, true, false)
    RELAX_AMD_SPLIT(7, true)
    RELAX_AMD_SPLIT(8, false)
    RELAX_AMD_SPLIT(12, true)
    RELAX_AMD_SPLIT(15, true)
    RELAX_AMD_SPLIT(16, false)
  }
  return RELAX_AMD_EUNSUPPORTED;
}
#undef RELAX_AMD_SPLIT_LDS
#undef RELAX_AMD_SPLIT_LDS_KERNEL
#undef RELAX_AMD_SPLIT
#undef RELAX_AMD_SPLIT_ROW
#undef RELAX_AMD_SPLIT_KERNEL


template int launch_actor_step_split<float>(const float*, int64_t, int64_t, int64_t, const int32_t*, const int32_t*,
                                            const int64_t*, float, const relax_amd_policy_loss_args&, float, float*,
                                            float*, float*, float*, float*, int64_t, hipStream_t);
template int launch_actor_step_split<bf16_t>(const bf16_t*, int64_t, int64_t, int64_t, const int32_t*, const int32_t*,
                                             const int64_t*, float, const relax_amd_policy_loss_args&, float, float*,
                                             float*, float*, float*, bf16_t*, int64_t, hipStream_t);
template int launch_actor_step_split<f16_t>(const f16_t*, int64_t, int64_t, int64_t, const int32_t*, const int32_t*,
                                            const int64_t*, float, const relax_amd_policy_loss_args&, float, float*,
                                            float*, float*, float*, f16_t*, int64_t, hipStream_t);

}  // namespace relax_amd


extern "C" int relax_amd_set_exchange_wait(int max_polls, int wait_tag_offset) {
  if (max_polls < 0 || wait_tag_offset < 0) {
    relax_amd::set_error("set_exchange_wait: negative argument");
    return RELAX_AMD_EINVAL;
  }
  relax_amd::g_max_polls.store(max_polls == 0 ? relax_amd::kWaitPolls : unsigned(max_polls), std::memory_order_relaxed);
  relax_amd::g_wait_tag_offset.store(unsigned(wait_tag_offset), std::memory_order_relaxed);
  return RELAX_AMD_OK;
}
