"""Tensor-level wrappers over the C ABI: argument checks, output allocation, stream hand-off, autograd glue.

PyTorch is used here only for device memory, streams and autograd bookkeeping; every arithmetic step on the token
path runs in the HIP kernels of ``librelax_amd.so``.
"""

from __future__ import annotations

import ctypes as C

import torch

from . import _lib
from ._lib import BF16, F16, F32, NUM_METRICS, check, lib, new_policy_loss_args

_DTYPE_CODES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}


def set_kernel_choice(name: str) -> str:
    """``relax_amd_set_kernel_choice``: "auto" | "two_walk" | "resident" for the entry points that hold two
    bit-identical kernels; returns the previous choice.  For tests and measurements."""
    from ._lib import KERNEL_CHOICES

    prev = lib.relax_amd_set_kernel_choice(KERNEL_CHOICES[name])
    if prev < 0:
        check(prev)
    return {v: k for k, v in KERNEL_CHOICES.items()}[prev]


_LAST_KERNEL: dict = {}


def _note_kernel(entry: str) -> None:
    _LAST_KERNEL[entry] = lib.relax_amd_last_kernel().decode()


def last_kernel(entry: str) -> str:
    """Which kernel family the last call of ``entry`` ("actor_step_fused" | "reverse_kl_step_fused" |
    "logprob_entropy_bwd") on this process launched (``relax_amd_last_kernel`` read right behind the call): e.g.
    "actor_step_split" for the one-shot workgroups, "actor_step_fused" for the two-walk kernel."""
    return _LAST_KERNEL.get(entry, "")


def _need_gpu(*tensors) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "relax_amd kernels run on a ROCm device only (got a CPU tensor); there is no CPU fallback"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} vs {t.device}")
    if dev is None:
        raise RuntimeError("relax_amd op called without any device tensor")
    return dev


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


# When set to a list, the big launches append (name, start_event, end_event) recorded on the launch stream, so a
# benchmark can read each kernel's duration without an external profiler.
kernel_events = None


class _timed:
    def __init__(self, name):
        self.name = name

    def __enter__(self):
        if kernel_events is not None:
            self.start = torch.cuda.Event(enable_timing=True)
            self.end = torch.cuda.Event(enable_timing=True)
            self.start.record()
        return self

    def __exit__(self, *exc):
        if kernel_events is not None:
            self.end.record()
            kernel_events.append((self.name, self.start, self.end))
        return False


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported logits dtype {t.dtype}; expected float32, bfloat16 or float16") from None


def _rows(t: torch.Tensor) -> torch.Tensor:
    """2-D view with unit inner stride (copy only if the caller handed something exotic)."""
    if t.dim() != 2:
        raise ValueError(f"expected a 2-D [rows, vocab] tensor, got shape {tuple(t.shape)}")
    if t.size(0) > 1 and t.size(1) > 0 and (t.stride(1) != 1 or t.stride(0) < t.size(1)):
        t = t.contiguous()
    elif t.size(1) > 0 and t.stride(1) != 1:
        t = t.contiguous()
    return t


def _f32(t, dev=None):
    if t is None:
        return None
    if t.dtype != torch.float32 or not t.is_contiguous():
        t = t.to(torch.float32).contiguous()
    return t


# ------------------------------------------------------------------------------------------------ log-prob / entropy


def logprob_entropy_fwd(logits, targets, row_ids=None, inv_temperature: float = 1.0, with_entropy: bool = True,
                        n_tokens: int | None = None):
    """Returns (log_prob, entropy | None, lse, spx | None), all fp32 [n_tokens]."""
    _need_gpu(logits, targets, row_ids)
    logits = _rows(logits)
    n = int(targets.numel()) if n_tokens is None else n_tokens
    if row_ids is None and n != logits.size(0):
        raise ValueError(f"{n} targets for {logits.size(0)} logits rows")
    if targets.dtype != torch.int64 or not targets.is_contiguous():
        targets = targets.to(torch.int64).contiguous()
    kw = dict(dtype=torch.float32, device=logits.device)
    lp = torch.empty(n, **kw)
    lse = torch.empty(n, **kw)
    ent = torch.empty(n, **kw) if with_entropy else None
    spx = torch.empty(n, **kw) if with_entropy else None
    with _timed("logprob_entropy_fwd"):
        check(lib.relax_amd_logprob_entropy_fwd(
            _p(logits), _code(logits), n, logits.size(1), logits.stride(0) if logits.size(0) > 1 else logits.size(1),
            _p(row_ids), _p(targets), float(inv_temperature), _p(lp), _p(ent), _p(lse), _p(spx), _stream()))
    return lp, ent, lse, spx


def logprob_entropy_bwd(logits, targets, lse, spx, g_lp, g_ent=None, token_of_row=None, grad_scale: float = 1.0,
                        grad_scale_dev=None, inv_temperature: float = 1.0, out=None):
    """dlogits [rows, vocab] in the logits dtype; every row is written."""
    _need_gpu(logits, targets, lse, g_lp)
    logits = _rows(logits)
    if out is None:
        out = torch.empty((logits.size(0), logits.size(1)), dtype=logits.dtype, device=logits.device)
    stride = logits.stride(0) if logits.size(0) > 1 else logits.size(1)
    g_lp, g_ent = _f32(g_lp), _f32(g_ent)
    with _timed("logprob_entropy_bwd"):
        check(lib.relax_amd_logprob_entropy_bwd(
            _p(logits), _code(logits), logits.size(0), logits.size(1), stride, _p(token_of_row), _p(targets), _p(lse),
            _p(spx), _p(g_lp), _p(g_ent), float(grad_scale), _p(grad_scale_dev), float(inv_temperature),
            _p(out), out.stride(0) if out.size(0) > 1 else out.size(1), _stream()))
    _note_kernel("logprob_entropy_bwd")
    return out


class LogProbEntropy(torch.autograd.Function):
    """(logits [R,V], targets [R]) -> (log_prob [R], entropy [R]); saves the logits reference + O(R) floats."""

    @staticmethod
    def forward(ctx, logits, targets, row_ids, token_of_row, inv_temperature, with_entropy, with_entropy_grad):
        with_entropy_grad = bool(with_entropy and with_entropy_grad)
        x = _rows(logits)
        if targets.dtype != torch.int64 or not targets.is_contiguous():
            targets = targets.to(torch.int64).contiguous()
        lp, ent, lse, spx = logprob_entropy_fwd(x, targets, row_ids, inv_temperature, with_entropy)
        ctx.save_for_backward(x, targets, lse, spx if with_entropy_grad else None, row_ids, token_of_row)
        ctx.inv_temperature = inv_temperature
        ctx.with_entropy_grad = with_entropy_grad
        if ent is None:
            ent = lp.new_zeros((0,))
        if not with_entropy_grad:
            ctx.mark_non_differentiable(ent)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        x, targets, lse, spx, row_ids, token_of_row = ctx.saved_tensors
        if g_lp is None:
            raise RuntimeError("LogProbEntropy expected a materialized grad_log_prob")
        if not ctx.with_entropy_grad or g_ent is None or g_ent.numel() == 0:
            g_ent = None
        if row_ids is not None and token_of_row is None:
            raise RuntimeError("row_ids without token_of_row cannot be differentiated")
        d = logprob_entropy_bwd(x, targets, lse, spx, g_lp.reshape(-1), None if g_ent is None else g_ent.reshape(-1),
                                token_of_row=token_of_row, inv_temperature=ctx.inv_temperature)
        return d, None, None, None, None, None, None


class LogProbEntropyMasked(torch.autograd.Function):
    """(logits [R,V], targets [R], keep mask bool [R,V]) -> (log_prob [R], entropy [R]): the log-prob's softmax is
    restricted to the kept vocabulary entries (plus the target), the entropy uses the whole row."""

    @staticmethod
    def forward(ctx, logits, targets, keep, inv_temperature, with_entropy, with_entropy_grad):
        with_entropy_grad = bool(with_entropy and with_entropy_grad)
        x = _rows(logits)
        n, v = x.shape
        if targets.dtype != torch.int64 or not targets.is_contiguous():
            targets = targets.to(torch.int64).contiguous()
        kw = dict(dtype=torch.float32, device=x.device)
        lp, lk = torch.empty(n, **kw), torch.empty(n, **kw)
        ent = torch.empty(n, **kw) if with_entropy else None
        lf = torch.empty(n, **kw) if with_entropy else None
        spx = torch.empty(n, **kw) if with_entropy else None
        stride = x.stride(0) if n > 1 else v
        check(lib.relax_amd_logprob_entropy_masked_fwd(_p(x), _code(x), n, v, stride, None, _p(targets), _p(keep), v,
                                                       float(inv_temperature), _p(lp), _p(ent), _p(lk), _p(lf),
                                                       _p(spx), _stream()))
        ctx.save_for_backward(x, targets, keep, lk, lf if with_entropy_grad else None,
                              spx if with_entropy_grad else None)
        ctx.inv_temperature = inv_temperature
        ctx.with_entropy_grad = with_entropy_grad
        if ent is None:
            ent = lp.new_zeros((0,))
        if not with_entropy_grad:
            ctx.mark_non_differentiable(ent)
        return lp, ent

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        x, targets, keep, lk, lf, spx = ctx.saved_tensors
        if g_lp is None:
            raise RuntimeError("LogProbEntropyMasked expected a materialized grad_log_prob")
        if not ctx.with_entropy_grad or g_ent is None or g_ent.numel() == 0:
            g_ent = None
        n, v = x.shape
        d = torch.empty((n, v), dtype=x.dtype, device=x.device)
        stride = x.stride(0) if n > 1 else v
        g_lp = _f32(g_lp.reshape(-1))
        g_ent = None if g_ent is None else _f32(g_ent.reshape(-1))
        check(lib.relax_amd_logprob_entropy_masked_bwd(_p(x), _code(x), n, v, stride, None, _p(targets), _p(keep), v,
                                                       _p(lk), _p(lf), _p(spx), _p(g_lp), _p(g_ent), 1.0,
                                                       float(ctx.inv_temperature), _p(d), v, _stream()))
        return d, None, None, None, None, None


# ------------------------------------------------------------------------------------------------------- row maps


def build_row_maps(row_begin, cu_resp, n_tokens: int, n_rows: int, want_inverse: bool = True):
    """row_begin [B] int64, cu_resp [B+1] int64 (device) -> (row_ids, sample_ids, token_of_row | None), int32."""
    dev = _need_gpu(row_begin, cu_resp)
    row_ids = torch.empty(n_tokens, dtype=torch.int32, device=dev)
    sample_ids = torch.empty(n_tokens, dtype=torch.int32, device=dev)
    inv = torch.empty(n_rows, dtype=torch.int32, device=dev) if want_inverse else None
    check(lib.relax_amd_build_row_maps(_p(row_begin), _p(cu_resp), row_begin.numel(), n_tokens, n_rows, _p(row_ids),
                                       _p(sample_ids), _p(inv), _stream()))
    return row_ids, sample_ids, inv


def gather_targets(packed_tokens, src_begin, src_end, cu_resp, out):
    """out[cu[i] + j] = packed_tokens[src_begin[i] + j] if that position is before src_end[i] else 0."""
    _need_gpu(packed_tokens, src_begin, src_end, cu_resp, out)
    check(lib.relax_amd_gather_targets(_p(packed_tokens), _p(src_begin), _p(src_end), _p(cu_resp), src_begin.numel(),
                                       _p(out), _stream()))
    return out


def segment_sum(mask, cu_resp, values=None):
    """fp64 [B]: per-sample sum of mask (or values*mask)."""
    dev = _need_gpu(mask, cu_resp)
    b = cu_resp.numel() - 1
    out = torch.empty(b, dtype=torch.float64, device=dev)
    check(lib.relax_amd_segment_sum(_p(_f32(values)), _p(_f32(mask)), _p(cu_resp), b, _p(out), _stream()))
    return out


# ---------------------------------------------------------------------------------------------------- policy loss


def _policy_args(*, n, advantages, loss_mask, cu_resp, log_prob=None, old_log_prob=None, ref_log_prob=None,
                 train_log_prob=None, rollout_log_prob=None, entropy=None, pg_loss_mask=None, sample_denom=None,
                 pg_sample_denom=None, loss_kind="ppo", kl_kind=None, unbiased_kl=False, use_opsm=False,
                 use_tis=False, mismatch_metrics=False, abs_diff_from_old=1, eps_clip=0.2, eps_clip_high=0.2,
                 eps_clip_c=None, entropy_coef=0.0, kl_coef=0.0, tis_lo=0.0, tis_hi=2.0, opsm_delta=1e-4,
                 tau_pos=1.0, tau_neg=1.05, per_token_outputs=False, want_coef_entropy=False,
                 extra_coef_log_prob=None, distill=None, topk_distill=None, read_masked_rows=False):
    """Fills a ``relax_amd_policy_loss_args`` block; returns (struct, outputs dict holding every live tensor).
    ``extra_coef_log_prob`` [n]: added to d loss / d log_prob of every unmasked token (the gradient of a caller's loss
    term that is linear in the log-probs).  ``distill`` = dict(teacher [n], kl_kind "k1" | "k3", min_clamp, token_clip,
    is_clip; None = off): ``extra_coef_log_prob`` then holds the weights of the sampled-token distillation signal and
    the kernel applies the signal's own derivative.  ``topk_distill`` = dict(ids int64 [n, K], teacher [n, K], width /
    valid int32 [n] | None, kl_mode, norm_mode, alpha, min_clamp, token_clip, is_clip; None = off; the fused step
    only): ``extra_coef_log_prob`` holds the weights of the top-K distillation signal, the step evaluates it next to
    each row's log-sum-exp and leaves ``topk_kl`` [n] and ``topk_grad`` [n, K] in the outputs.  ``read_masked_rows``
    (the fused step only): rows of fully masked tokens are scanned too, so their log-probs, entropies and distillation
    signals are real instead of 0."""
    dev = _need_gpu(advantages, loss_mask, cu_resp)
    b = int(cu_resp.numel()) - 1
    if loss_kind not in _lib.LOSS_KINDS:
        raise ValueError(f"unknown loss kind {loss_kind}")
    if kl_kind not in _lib.KL_KINDS:
        raise ValueError(f"Unknown kl_loss_type: {kl_kind}")
    if cu_resp.dtype != torch.int64:
        raise TypeError("cu_resp must be int64")
    keep = [_f32(t) for t in (log_prob, old_log_prob, ref_log_prob, train_log_prob, rollout_log_prob, advantages,
                               loss_mask, pg_loss_mask, entropy, sample_denom, pg_sample_denom)]
    extra = _f32(extra_coef_log_prob)
    for t in keep[:9] + [extra]:
        if t is not None and t.numel() != n:
            raise ValueError(f"per-token tensor has {t.numel()} elements, expected {n}")
    for t in keep[9:]:
        if t is not None and t.numel() != b:
            raise ValueError(f"per-sample denominator has {t.numel()} elements, expected {b}")
    kw = dict(dtype=torch.float32, device=dev)
    out = {
        "coef_log_prob": torch.empty(n, **kw),
        "coef_entropy": torch.empty(n, **kw) if (entropy is not None or want_coef_entropy) else None,
        "metrics": torch.empty(NUM_METRICS, **kw),
    }
    if per_token_outputs:
        for k in ("pg_loss_tok", "clipfrac_tok", "ppo_kl_tok"):
            out[k] = torch.empty(n, **kw)
        out["kl_tok"] = torch.empty(n, **kw) if kl_kind is not None else None
    partials = torch.empty(max(b, 1) * NUM_METRICS, **kw)
    a = new_policy_loss_args()
    (a.log_prob, a.old_log_prob, a.ref_log_prob, a.train_log_prob, a.rollout_log_prob, a.advantages, a.loss_mask,
     a.pg_loss_mask, a.entropy, a.sample_denom, a.pg_sample_denom) = [None if t is None else t.data_ptr() for t in keep]
    a.cu_resp = cu_resp.data_ptr()
    a.n_samples, a.n_tokens = b, n
    a.loss_kind, a.kl_kind = _lib.LOSS_KINDS[loss_kind], _lib.KL_KINDS[kl_kind]
    a.unbiased_kl, a.use_opsm, a.use_tis = int(unbiased_kl), int(use_opsm), int(use_tis)
    a.mismatch_metrics, a.abs_diff_from_old = int(mismatch_metrics), int(abs_diff_from_old)
    a.eps_clip, a.eps_clip_high = float(eps_clip), float(eps_clip_high)
    a.eps_clip_c = -1.0 if eps_clip_c is None else float(eps_clip_c)
    a.entropy_coef, a.kl_coef = float(entropy_coef), float(kl_coef)
    a.tis_lo, a.tis_hi, a.opsm_delta = float(tis_lo), float(tis_hi), float(opsm_delta)
    a.tau_pos, a.tau_neg = float(tau_pos), float(tau_neg)
    a.coef_log_prob = out["coef_log_prob"].data_ptr()
    a.coef_entropy = None if out["coef_entropy"] is None else out["coef_entropy"].data_ptr()
    for k in ("pg_loss_tok", "clipfrac_tok", "ppo_kl_tok", "kl_tok"):
        t = out.get(k)
        setattr(a, k, None if t is None else t.data_ptr())
    a.sample_partials = partials.data_ptr()
    a.metrics = out["metrics"].data_ptr()
    a.extra_coef_log_prob = None if extra is None else extra.data_ptr()
    teacher = None
    if distill is not None:
        teacher = _f32(distill["teacher"])
        if extra is None or teacher.numel() != n:
            raise ValueError("distill needs extra_coef_log_prob and a teacher log-prob per token")
        a.distill_teacher_log_prob = teacher.data_ptr()
        a.distill_kl_kind = _lib.KL_KINDS[distill["kl_kind"]]
        nan = float("nan")
        a.distill_min_clamp, a.distill_token_clip, a.distill_is_clip = (
            nan if distill.get(k) is None else float(distill[k]) for k in ("min_clamp", "token_clip", "is_clip"))
    a.read_masked_rows = int(bool(read_masked_rows))
    held = None
    if topk_distill is not None:
        td = topk_distill
        ids, t_lp = td["ids"], _f32(td["teacher"])
        k = int(ids.size(1)) if ids.dim() == 2 else 0
        if extra is None or distill is not None or ids.dtype != torch.int64 or tuple(ids.shape) != (n, k) \
                or tuple(t_lp.shape) != (n, k) or not (1 <= k <= _lib.FUSED_TOPK_MAX):
            raise ValueError("topk_distill needs extra_coef_log_prob, no sampled-token distill block, int64 ids "
                             f"[n, K] and teacher log-probs of the same shape, 1 <= K <= {_lib.FUSED_TOPK_MAX}")
        ids, t_lp = ids.contiguous(), t_lp.contiguous()
        per_tok = []
        for key in ("width", "valid"):
            v = td.get(key)
            if v is not None:
                if v.dtype != torch.int32 or v.numel() != n:
                    raise ValueError(f"topk_distill[{key!r}] must be int32 [n]")
                v = v.contiguous()
            per_tok.append(v)
        out["topk_kl"] = torch.zeros(n, **kw)
        out["topk_grad"] = torch.zeros((n, k), **kw)
        a.topk_ids, a.topk_teacher_log_prob = ids.data_ptr(), t_lp.data_ptr()
        a.topk_width, a.topk_valid = (None if v is None else v.data_ptr() for v in per_tok)
        a.topk_k, a.topk_kl_mode, a.topk_norm_mode = k, int(td["kl_mode"]), int(td["norm_mode"])
        a.topk_jsd_alpha = float(td["alpha"])
        clamp = td.get("min_clamp")
        a.topk_has_clamp, a.topk_min_clamp = (0, 0.0) if clamp is None else (1, float(clamp))
        nan = float("nan")
        a.distill_min_clamp = nan
        a.distill_token_clip, a.distill_is_clip = (
            nan if td.get(key) is None else float(td[key]) for key in ("token_clip", "is_clip"))
        a.topk_kl, a.topk_grad = out["topk_kl"].data_ptr(), out["topk_grad"].data_ptr()
        held = (ids, t_lp, per_tok)
    out["_keepalive"] = (keep, partials, cu_resp, extra, teacher, held)
    return a, out


def policy_loss(*, log_prob, **kw):
    """Runs the two policy-loss launches.  Returns dict(metrics [16], coef_log_prob, coef_entropy, per-token...)."""
    _need_gpu(log_prob)
    a, out = _policy_args(n=int(log_prob.numel()), log_prob=log_prob, **kw)
    check(lib.relax_amd_policy_loss(C.byref(a), _stream()))
    return out


def actor_step_fused(logits, targets, token_of_row, sample_ids, n_tokens: int, inv_temperature: float,
                     grad_scale: float = 1.0, **kw):
    """One launch: log-prob + entropy forward, per-token loss coefficients and dlogits; then the policy-loss launches
    for the metrics.  Returns (out dict as policy_loss, log_prob, entropy, lse, spx, dlogits)."""
    dev = _need_gpu(logits, targets)
    logits = _rows(logits)
    if targets.dtype != torch.int64 or not targets.is_contiguous():
        targets = targets.to(torch.int64).contiguous()
    f = dict(dtype=torch.float32, device=dev)
    lp, ent, lse, spx = (torch.empty(n_tokens, **f) for _ in range(4))
    dlogits = torch.empty((logits.size(0), logits.size(1)), dtype=logits.dtype, device=dev)
    a, out = _policy_args(n=n_tokens, want_coef_entropy=True, **kw)
    stride = logits.stride(0) if logits.size(0) > 1 else logits.size(1)
    with _timed("actor_step_fused"):
        check(lib.relax_amd_actor_step_fused(
            _p(logits), _code(logits), logits.size(0), logits.size(1), stride, _p(token_of_row), _p(sample_ids),
            _p(targets), float(inv_temperature), C.byref(a), float(grad_scale), _p(lp), _p(ent), _p(lse), _p(spx),
            _p(dlogits), logits.size(1), _stream()))
    _note_kernel("actor_step_fused")
    a.log_prob, a.entropy = lp.data_ptr(), ent.data_ptr()
    check(lib.relax_amd_policy_loss(C.byref(a), _stream()))
    return out, lp, ent, lse, spx, dlogits


def sparse_row_add(dlogits, row_ids, ids, values, targets=None, target_values=None, scale: float = 1.0):
    """``dlogits[row_ids[t], ids[t, j]] += values[t, j] * scale`` (and the same at ``targets[t]`` with
    ``target_values[t]``), in place; ids outside the vocabulary are skipped."""
    _need_gpu(dlogits, ids)
    d = dlogits.reshape(-1, dlogits.size(-1))
    n, k = ids.shape
    stride = d.stride(0) if d.size(0) > 1 else d.size(1)
    check(lib.relax_amd_sparse_row_add(_p(d), _code(d), n, d.size(1), stride, _p(row_ids), _p(ids.contiguous()),
                                       _p(_f32(values)), k, _p(targets), _p(_f32(target_values)), float(scale),
                                       _stream()))
    return dlogits


TOPK_ROWS_MAX_K = 512
TOPK_ROWS_MAX_VOCAB = 1000000


def topk_rows(logits, row_ids, k: int, with_values: bool = True):
    """The ``k`` largest logits of each token's row, largest first: ``(values fp32 [n, k] | None, indices int64
    [n, k])``.  ``row_ids`` (int32 [n]) names the logits row of each token; None scores every row."""
    dev = _need_gpu(logits)
    logits = _rows(logits)
    n = int(row_ids.numel()) if row_ids is not None else logits.size(0)
    k = int(k)
    values = torch.empty((n, k), dtype=torch.float32, device=dev) if with_values else None
    indices = torch.empty((n, k), dtype=torch.int64, device=dev)
    flags = torch.empty(max(n, 1), dtype=torch.uint8, device=dev)
    stride = logits.stride(0) if logits.size(0) > 1 else logits.size(1)
    with _timed("topk_rows"):
        check(lib.relax_amd_topk_rows(_p(logits), _code(logits), n, logits.size(1), stride, _p(row_ids), k, _p(values),
                                      _p(indices), _p(flags), _stream()))
    return values, indices


def logprob_entropy_topk_fwd(logits, targets, row_ids, inv_temperature: float, k: int, with_entropy: bool = True,
                             with_values: bool = False):
    """``logprob_entropy_fwd`` and ``topk_rows`` over the same rows from one read of the logits.  Returns
    ``(log_prob, entropy | None, lse, spx | None, values | None, indices)``."""
    dev = _need_gpu(logits, targets, row_ids)
    logits = _rows(logits)
    n = int(targets.numel())
    if row_ids is None and n != logits.size(0):
        raise ValueError(f"{n} targets for {logits.size(0)} logits rows")
    if targets.dtype != torch.int64 or not targets.is_contiguous():
        targets = targets.to(torch.int64).contiguous()
    k = int(k)
    kw = dict(dtype=torch.float32, device=dev)
    lp, lse = torch.empty(n, **kw), torch.empty(n, **kw)
    ent = torch.empty(n, **kw) if with_entropy else None
    spx = torch.empty(n, **kw) if with_entropy else None
    values = torch.empty((n, k), **kw) if with_values else None
    indices = torch.empty((n, k), dtype=torch.int64, device=dev)
    flags = torch.empty(max(n, 1), dtype=torch.uint8, device=dev)
    stride = logits.stride(0) if logits.size(0) > 1 else logits.size(1)
    with _timed("logprob_entropy_topk_fwd"):
        check(lib.relax_amd_logprob_entropy_topk_fwd(
            _p(logits), _code(logits), n, logits.size(1), stride, _p(row_ids), _p(targets), float(inv_temperature), k,
            _p(lp), _p(ent), _p(lse), _p(spx), _p(values), _p(indices), _p(flags), _stream()))
    return lp, ent, lse, spx, values, indices


def scale_rows_inplace(data, factor_dev):
    data2 = data.reshape(-1, data.size(-1))
    stride = data2.stride(0) if data2.size(0) > 1 else data2.size(1)
    check(lib.relax_amd_scale_rows_inplace(_p(data2), _code(data2), data2.size(0), data2.size(1), stride,
                                           _p(factor_dev), _stream()))
    return data


# ----------------------------------------------------------------------------------------------------- advantages


def group_rewards(rewards, group_index, mode: str):
    """rewards fp32|fp64 [B], group_index int32 [B] (device) -> (normalised [B] same dtype, group sizes int32 [B])."""
    dev = _need_gpu(rewards, group_index)
    n = int(rewards.numel())
    if rewards.dtype not in (torch.float32, torch.float64):
        rewards = rewards.float()
    rewards = rewards.contiguous()
    out = torch.empty(n, dtype=rewards.dtype, device=dev)
    cnt = torch.empty(n, dtype=torch.int32, device=dev)
    code = _lib.F32 if rewards.dtype == torch.float32 else _lib.F64
    check(lib.relax_amd_group_rewards(_p(rewards), code, _p(group_index.to(torch.int32).contiguous()), n,
                                      _lib.GROUP_MODES[mode], _p(out), _p(cnt), _stream()))
    return out, cnt


def broadcast_per_sample(per_sample, cu_resp, n_tokens: int):
    dev = _need_gpu(per_sample, cu_resp)
    out = torch.empty(n_tokens, dtype=torch.float32, device=dev)
    check(lib.relax_amd_broadcast_per_sample(_p(_f32(per_sample)), _p(cu_resp), cu_resp.numel() - 1, _p(out),
                                             _stream()))
    return out


def masked_whiten(values, mask, shift_mean: bool = True, epsilon: float = 1e-8):
    """Returns (whitened fp32 [N], stats fp32 [4] = sum, sum of squares, mask sum, rstd)."""
    dev = _need_gpu(values, mask)
    n = int(values.numel())
    if n == 0:
        raise ValueError("masked_whiten needs at least one value")
    v, m = _f32(values.reshape(-1)), _f32(mask.reshape(-1))
    partials = torch.empty(3 * lib.relax_amd_whiten_partials(n), dtype=torch.float64, device=dev)
    stats = torch.empty(4, dtype=torch.float32, device=dev)
    out = torch.empty(n, dtype=torch.float32, device=dev)
    check(lib.relax_amd_masked_whiten(_p(v), _p(m), n, int(shift_mean), float(epsilon), _p(partials), _p(stats),
                                      _p(out), _stream()))
    return out, stats


# ------------------------------------------------------------------------------------------------------ reverse KL


def reverse_kl_fwd(student, teacher):
    _need_gpu(student, teacher)
    s, t = _rows(student), _rows(teacher)
    if s.shape != t.shape or s.dtype != t.dtype:
        raise ValueError(f"student {tuple(s.shape)}/{s.dtype} and teacher {tuple(t.shape)}/{t.dtype} must match")
    if s.size(0) > 1 and s.stride(0) != t.stride(0):
        s, t = s.contiguous(), t.contiguous()
    n = s.size(0)
    kw = dict(dtype=torch.float32, device=s.device)
    kl, ls, lt = torch.empty(n, **kw), torch.empty(n, **kw), torch.empty(n, **kw)
    stride = s.stride(0) if n > 1 else s.size(1)
    with _timed("reverse_kl_fwd"):
        check(lib.relax_amd_reverse_kl_fwd(_p(s), _p(t), _code(s), n, s.size(1), stride, _p(kl), _p(ls), _p(lt),
                                           _stream()))
    return kl, ls, lt, s, t


def reverse_kl_bwd(s, t, kl, ls, lt, g, grad_scale: float = 1.0, grad_scale_dev=None):
    n = s.size(0)
    stride = s.stride(0) if n > 1 else s.size(1)
    if stride != s.size(1):
        raise ValueError("reverse_kl_bwd writes a dense gradient: student rows must be contiguous")
    d = torch.empty_like(s)
    g = _f32(g)
    with _timed("reverse_kl_bwd"):
        check(lib.relax_amd_reverse_kl_bwd(_p(s), _p(t), _code(s), n, s.size(1), stride, _p(kl), _p(ls), _p(lt),
                                           _p(g), float(grad_scale), _p(grad_scale_dev), _p(d), _stream()))
    return d


def reverse_kl_step_fused(student, teacher, g, grad_scale: float = 1.0):
    """One launch: (kl, lse_s, lse_t, dstudent) with ``dstudent = g[t] * grad_scale * d kl[t] / d student``."""
    _need_gpu(student, teacher, g)
    s, t = _rows(student), _rows(teacher)
    if s.shape != t.shape or s.dtype != t.dtype:
        raise ValueError(f"student {tuple(s.shape)}/{s.dtype} and teacher {tuple(t.shape)}/{t.dtype} must match")
    if s.size(0) > 1 and (s.stride(0) != s.size(1) or t.stride(0) != t.size(1)):
        s, t = s.contiguous(), t.contiguous()
    n = s.size(0)
    g = _f32(g)
    if g.numel() != n:
        raise ValueError(f"g has {g.numel()} entries for {n} token rows")
    kw = dict(dtype=torch.float32, device=s.device)
    kl, ls, lt = torch.empty(n, **kw), torch.empty(n, **kw), torch.empty(n, **kw)
    d = torch.empty_like(s)
    with _timed("reverse_kl_step_fused"):
        check(lib.relax_amd_reverse_kl_step_fused(_p(s), _p(t), _code(s), n, s.size(1), s.size(1), _p(g),
                                                  float(grad_scale), _p(kl), _p(ls), _p(lt), _p(d), _stream()))
    _note_kernel("reverse_kl_step_fused")
    return kl, ls, lt, d


class ReverseKL(torch.autograd.Function):
    """(student logits [R,V], teacher logits [R,V]) -> per-token KL(student || teacher) [R]; teacher gets no grad."""

    @staticmethod
    def forward(ctx, student, teacher):
        kl, ls, lt, s, t = reverse_kl_fwd(student, teacher)
        if s.size(0) > 1 and s.stride(0) != s.size(1):
            s, t = s.contiguous(), t.contiguous()
        ctx.save_for_backward(s, t, kl, ls, lt)
        return kl

    @staticmethod
    def backward(ctx, g):
        s, t, kl, ls, lt = ctx.saved_tensors
        return reverse_kl_bwd(s, t, kl, ls, lt, g.reshape(-1)), None
