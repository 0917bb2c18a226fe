// Register-resident fused actor step for fp32 rows too long to sit in the registers as fp32: rows of 100352 ..
// 163840 entries, the vocabularies a stock Megatron model hands a custom loss as fp32 [1, T, V] logits
// (relax/backends/megatron/loss.py:92-97 asserts the dtype).  Same computation, same outputs, bit for bit, as
// actor_step_fused_kernel<float> (log-prob + entropy forward, per-token policy-loss coefficients, dlogits backward;
// _VocabParallelLogProbEntropy.forward + .backward, relax/utils/training/ppo_utils.py:481-629, and the per-token part
// of policy_loss_function, loss.py:961-1100).
//
// Such logits are a bf16 output layer's values widened by `.float()`: the low 16 bits of every word are zero.  A
// 1024-thread workgroup therefore keeps the row as the upper halves only (V = 151936: 38 four-float vectors per thread
// packed into 19 registers-quads, the footprint of a bf16 row) and checks on the way that nothing was dropped.  A row
// that passes the check is read from HBM once: its gradient is computed from the registers.  A row that does not (fp32
// logits with real low bits) takes its values from memory again in the gradient pass, as the two-walk kernel does --
// the result is the same for every input, only the traffic differs.
//
// The softmax scan runs on the fp32 values as they land, in scan_row()'s grouping and order (four vectors absorbed
// together while a thread has four to go, then single vectors; waves merged in index order), so log-probs are
// bit-identical to the forward-only kernel's.  Workgroups are persistent, one per CU; no workgroup waits for another
// and the loop bound is the only exit condition.
//
// hipcc-flags: -mllvm -amdgpu-use-amdgpu-trackers=1
#include "actor_step_resident.h"

#include "device_utils.h"
#include "loss_math.h"
#include "row_scan.h"

namespace relax_amd {

namespace {

constexpr int kWideThreads = 1024;

// upper halves of two four-float vectors, in memory order
__device__ __forceinline__ u32x4 wide_pack(const u32x4& a, const u32x4& b) {
  return u32x4{(a.x >> 16) | (a.y & 0xffff0000u), (a.z >> 16) | (a.w & 0xffff0000u), (b.x >> 16) | (b.y & 0xffff0000u),
               (b.z >> 16) | (b.w & 0xffff0000u)};
}
__device__ __forceinline__ uint32_t wide_low_bits(const u32x4& a) { return (a.x | a.y | a.z | a.w) & 0xffffu; }
// vector `half` (0 / 1) of a packed pair, widened again
__device__ __forceinline__ void wide_unpack(const u32x4& r, int half, float (&o)[4]) {
  const uint32_t w0 = half ? r.z : r.x, w1 = half ? r.w : r.y;
  o[0] = __uint_as_float(w0 << 16);
  o[1] = __uint_as_float(w0 & 0xffff0000u);
  o[2] = __uint_as_float(w1 << 16);
  o[3] = __uint_as_float(w1 & 0xffff0000u);
}

struct WideTokenData {
  TokenInputs in;
  float x_target, den, pg_den;
  int64_t tg;
};

}  // namespace

// NF full vector positions per thread plus one partially filled position when PARTIAL.  Positions are packed in pairs;
// with an odd count the last register quad is half used.
template <int NF, bool PARTIAL>
__global__ __launch_bounds__(kWideThreads, 4) void actor_step_resident_wide_kernel(
    const float* __restrict__ logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
    const int32_t* __restrict__ token_of_row, const int32_t* __restrict__ sample_ids,
    const int64_t* __restrict__ targets, float c, float inv_t, relax_amd_policy_loss_args a, float grad_scale,
    float* __restrict__ log_prob, float* __restrict__ entropy, float* __restrict__ lse_out,
    float* __restrict__ spx_out, float* __restrict__ dlogits, int64_t d_stride) {
  constexpr int THREADS = kWideThreads, kU = kScanUnroll;
  constexpr int NP = NF + (PARTIAL ? 1 : 0);  // vector positions per thread
  static_assert(kU == 4, "positions are packed in pairs and scanned in groups of four");
  constexpr int NR = (NP + 1) / 2;            // packed registers-quads
  constexpr int kGroups = (NP + kU - 1) / kU;
  __shared__ float wave_state[THREADS / kWave][3];
  __shared__ uint32_t wave_inexact[THREADS / kWave];
  __shared__ float bc[6];
  __shared__ int64_t bc_target;
  const int tid = threadIdx.x;
  const bool wave0 = __builtin_amdgcn_readfirstlane(tid) < kWave;
  const int rem = int(vocab / 4) - NF * THREADS;  // lanes that hold a vector at the partial position (host-checked)
  u32x4 reg[NR];

  auto has = [&](int p) -> bool { return p < NF || (PARTIAL && p == NF && tid < rem); };
  auto live_token = [&](int64_t row) -> int64_t {
    if (row >= n_rows) return -1;
    const int64_t tok = token_of_row ? int64_t(token_of_row[row]) : row;
    if (tok < 0) return -1;
    const float m = a.loss_mask[tok];
    const float mp = a.pg_loss_mask ? a.pg_loss_mask[tok] : m;
    return (m == 0.f && mp == 0.f && !a.read_masked_rows) ? -1 : tok;
  };
  auto fetch_token = [&](int64_t row, int64_t tok) {
    WideTokenData td{};
    td.tg = -1;
    if (wave0 && tok >= 0) {
      if (tid == 0) {
        td.in = load_token_inputs(a, tok);
        td.tg = targets[tok];
        if (td.tg >= 0 && td.tg < vocab) td.x_target = logits[row * row_stride + td.tg];
        const int32_t sid = sample_ids ? sample_ids[tok] : 0;
        td.den = a.sample_denom ? a.sample_denom[sid] : 1.0f;
        td.pg_den = a.pg_sample_denom ? a.pg_sample_denom[sid] : td.den;
      }
    }
    return td;
  };
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
    for (int p = 0; p < NP; ++p)
      if (has(p)) store_stream(dv + tid + p * THREADS, u32x4{0u, 0u, 0u, 0u});
  };
  auto advance = [&](int64_t row) -> int64_t {
    while (row < n_rows && live_token(row) < 0) {
      zero_row(row);
      row += gridDim.x;
    }
    return row;
  };

  // A live row arrives: group by group (four positions = one scan group) the vectors land in `land`, are absorbed into
  // the softmax state as the fp32 values they are, and leave their upper halves in `reg`.  The loads of the following
  // group are requested before a group is absorbed.  Returns the OR of the low halves this lane saw.
  auto load_and_scan = [&](int64_t row, SoftmaxAcc& st) -> uint32_t {
    const u32x4* xv = reinterpret_cast<const u32x4*>(logits + row * row_stride);
    u32x4 land[2][kU];
    uint32_t low = 0u;
    bool grouped = true;
    auto request = [&](int g) {
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int p = kU * g + u;
        int lane_id = tid;
        asm volatile("" : "+v"(lane_id));
        land[g & 1][u] = (p < NP && has(p)) ? load_stream(xv + lane_id + p * THREADS) : u32x4{0u, 0u, 0u, 0u};
      }
    };
    request(0);
#pragma unroll
    for (int g = 0; g < kGroups; ++g) {
      if (g + 1 < kGroups) request(g + 1);
      u32x4(&l)[kU] = land[g & 1];
      if (grouped && kU * g + kU - 1 < NP && has(kU * g + kU - 1)) {
        float v[kU * 4];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          float part[4];
          Row<float>::unpack(l[u], part);
#pragma unroll
          for (int k = 0; k < 4; ++k) v[u * 4 + k] = part[k];
        }
        scan_absorb(v, c, st);
      } else {
        grouped = false;
#pragma unroll
        for (int u = 0; u < kU; ++u)
          if (kU * g + u < NP && has(kU * g + u)) {
            float v[4];
            Row<float>::unpack(l[u], v);
            scan_absorb(v, c, st);
          }
      }
#pragma unroll
      for (int u = 0; u < kU; u += 2)
        if (kU * g + u < NP) {
          low |= wide_low_bits(l[u]) | wide_low_bits(l[u + 1]);
          u32x4 r = wide_pack(l[u], l[u + 1]);
          // packed here and now: left to itself the compiler parks the landed vectors in scratch memory and packs
          // them when the gradient pass first asks for the result
          asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w), "+v"(low));
          reg[(kU * g + u) / 2] = r;
        }
      asm volatile("" : "+v"(st.m), "+v"(st.s), "+v"(st.t));
      __builtin_amdgcn_sched_barrier(0);
    }
    return low;
  };

  int64_t row = advance(blockIdx.x);
  if (row >= n_rows) return;
  int64_t tok = live_token(row);
  SoftmaxAcc st{kNegHuge, 0.f, 0.f};
  uint32_t low = load_and_scan(row, st);

  while (true) {
    const int64_t next = advance(row + gridDim.x);
    const bool has_next = next < n_rows;
    const int64_t next_tok = has_next ? live_token(next) : -1;
    const WideTokenData td = fetch_token(row, tok);
    // did any lane of the workgroup drop non-zero low halves?  One word per wave, read by thread 0 behind the barrier
    // of the merge below.
    {
      const bool any = __builtin_amdgcn_ballot_w64(low != 0u) != 0ull;
      if ((tid & (kWave - 1)) == 0) wave_inexact[tid / kWave] = any ? 1u : 0u;
    }
    scan_block_merge<THREADS>(st, wave_state);
    if (wave0) {
      if (tid == 0) {
        float lse = 0.f, spx = 0.f, ent = 0.f, lp = 0.f;
        scan_finish(st, td.x_target, td.tg >= 0 && td.tg < vocab, inv_t, lse, spx, ent, lp);
        log_prob[tok] = lp;
        entropy[tok] = ent;
        lse_out[tok] = lse;
        spx_out[tok] = spx;
        relax_amd_policy_loss_args al = a;
        asm volatile("" : "+s"(al.eps_clip), "+s"(al.eps_clip_high), "+s"(al.eps_clip_c), "+s"(al.entropy_coef),
                     "+s"(al.kl_coef), "+s"(al.tis_lo), "+s"(al.tis_hi), "+s"(al.tau_pos), "+s"(al.tau_neg));
        const TokenResult tr = token_terms(al, td.in, lp, ent, false, 0.f, td.den, td.pg_den);
        a.coef_log_prob[tok] = tr.coef_lp;
        if (a.coef_entropy) a.coef_entropy[tok] = tr.coef_ent;
        const float glp = tr.coef_lp * grad_scale, gh = tr.coef_ent * grad_scale;
        const float b = gh * inv_t;
        uint32_t inexact = 0u;
#pragma unroll
        for (int w = 0; w < THREADS / kWave; ++w) inexact |= wave_inexact[w];
        bc[0] = -lse * kLog2e;           // k0: p = exp2(x*c + k0)
        bc[1] = -glp * inv_t + b * spx;  // a0
        bc[2] = -b * inv_t;              // a1: d = p * (a0 + a1*x)
        bc[3] = glp * inv_t;             // added at the target
        bc[4] = (glp == 0.f && gh == 0.f) ? 1.f : 0.f;
        bc[5] = inexact ? 1.f : 0.f;
        bc_target = td.tg;
      }
    }
    __syncthreads();
    const float k0 = bc[0], a0 = bc[1], a1 = bc[2], hot = bc[3];
    const int64_t tg = bc_target;
    const bool emit_zero = bc[4] != 0.f;
    const bool reread = bc[5] != 0.f;  // uniform over the workgroup

    u32x4* dv = reinterpret_cast<u32x4*>(dlogits + row * d_stride);
    const u32x4* xv = reinterpret_cast<const u32x4*>(logits + row * row_stride);
    const int tvec = (tg >= 0 && tg < vocab) ? int(tg / 4) : -1;
    const int tsub = int(tg % 4);
    auto gradient_of = [&](float (&v)[4], int idx) {
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k] = fast_exp2(fmaf(v[k], c, k0)) * fmaf(v[k], a1, a0);
      if (idx == tvec) {  // one lane of the workgroup per row
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (k == tsub) v[k] += hot;
      }
    };
    if (emit_zero) {
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        int lane_id = tid;
        asm volatile("" : "+v"(lane_id));
        if (has(p)) store_stream(dv + lane_id + p * THREADS, u32x4{0u, 0u, 0u, 0u});
      }
    } else if (!reread) {
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        int lane_id = tid;
        asm volatile("" : "+v"(lane_id));
        const int idx = lane_id + p * THREADS;
        float v[4];
        wide_unpack(reg[p / 2], p & 1, v);
        gradient_of(v, idx);
        if (has(p)) store_stream(dv + idx, Row<float>::pack(v));
        __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      // the registers hold rounded values: this row's own words come from memory once more, four positions at a time
#pragma unroll
      for (int g = 0; g < kGroups; ++g) {
        u32x4 raw[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const int p = kU * g + u;
          int lane_id = tid;
          asm volatile("" : "+v"(lane_id));
          if (p < NP) raw[u] = has(p) ? load_stream(xv + lane_id + p * THREADS) : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
          const int p = kU * g + u;
          if (p < NP) {
            int lane_id = tid;
            asm volatile("" : "+v"(lane_id));
            const int idx = lane_id + p * THREADS;
            float v[4];
            Row<float>::unpack(raw[u], v);
            gradient_of(v, idx);
            if (has(p)) store_stream(dv + idx, Row<float>::pack(v));
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (!has_next) return;
    st = SoftmaxAcc{kNegHuge, 0.f, 0.f};
    low = load_and_scan(next, st);
    row = next;
    tok = next_tok;
  }
}

#define RELAX_AMD_WIDE(NF, PARTIAL)                                                                                  \
  if (full == NF && partial == PARTIAL) {                                                                             \
    hipLaunchKernelGGL((actor_step_resident_wide_kernel<NF, PARTIAL>), grid, block, 0, stream, logits, row_stride,   \
                       vocab, n_rows, token_of_row, sample_ids, targets, inv_t * kLog2e, inv_t, a, grad_scale,       \
                       log_prob, entropy, lse, spx, dlogits, d_stride);                                              \
    return check_launch("actor_step_resident_wide");                                                                 \
  }

int launch_actor_step_resident_wide(const float* logits, int64_t row_stride, int64_t vocab, int64_t n_rows,
                                    const int32_t* token_of_row, const int32_t* sample_ids, const int64_t* targets,
                                    float inv_t, const relax_amd_policy_loss_args& a, float grad_scale,
                                    float* log_prob, float* entropy, float* lse, float* spx, float* dlogits,
                                    int64_t d_stride, int compute_units, hipStream_t stream) {
  // the top-K distillation block is evaluated by the two-walk kernel for these rows
  if (a.topk_ids || vocab % 4 != 0 || scan_threads(vocab, 4) != kWideThreads) return RELAX_AMD_EUNSUPPORTED;
  const int64_t nvec = vocab / 4;
  const int full = int(nvec / kWideThreads);
  const bool partial = nvec % kWideThreads != 0;
  const dim3 grid(static_cast<unsigned>(n_rows < compute_units ? n_rows : compute_units)), block(kWideThreads);
  // 151936 / 152064 (37984 / 38016 vectors), 128256 / 129280 (32064 / 32320), 131072 (32768), 163840 (40960),
  // 100352 / 102400 (25088 / 25600)
  RELAX_AMD_WIDE(37, true)
  RELAX_AMD_WIDE(31, true)
  RELAX_AMD_WIDE(32, false)
  RELAX_AMD_WIDE(40, false)
  RELAX_AMD_WIDE(24, true)
  RELAX_AMD_WIDE(25, false)
  return RELAX_AMD_EUNSUPPORTED;
}
#undef RELAX_AMD_WIDE

}  // namespace relax_amd
