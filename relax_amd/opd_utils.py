"""On-policy-distillation KL on full-vocabulary logits (gfx950 kernels) and the reference's token-mean reduction.

``compute_opd_kl_full_vocab`` is the K = vocab case of ``compute_opd_kl``'s ``jsd_alpha == 0`` branch
(relax/utils/opd/opd_utils.py:1097-1228) evaluated straight from logits, so the [N, V] log-softmax tensors of the
student and the teacher are never materialised.  ``reduce_opd_loss`` follows :1355-1365.
"""

from __future__ import annotations

import torch

from . import _lib, ops
from ._lib import check, lib
from .cp_utils import _cu
from .ops import _code, _f32, _need_gpu, _p, _rows, _stream

OPD_KL_TYPES = ("reverse_kl", "forward_kl", "jsd", "low_var_kl")
_NORM_MODES = {"tail": 0, "norm": 1, "trunc": 2}


def compute_opd_kl_full_vocab(student_logits: torch.Tensor, teacher_logits: torch.Tensor) -> torch.Tensor:
    """Per-token reverse KL(student || teacher) over the whole vocabulary, fp32 [N]; differentiable w.r.t. the
    student logits (the teacher is treated as detached, as the reference detaches teacher log-probs)."""
    return ops.ReverseKL.apply(student_logits, teacher_logits.detach())


class TopKLogProbs(torch.autograd.Function):
    """(logits [T, V], ids int64 [N, K]) -> log-probs [N, K] fp32 at the given vocabulary ids.  ``row_ids`` /
    ``token_of_row`` (int32, optional) map the N tokens to logits rows and back for the packed response layout; without
    them token t is row t.  Saves the logits reference, the ids and one float per token; the backward writes the
    dense [T, V] gradient in one streaming pass."""

    @staticmethod
    def forward(ctx, logits, ids, inv_temperature, lse, row_ids=None, token_of_row=None, differentiable=True):
        x = _rows(logits)
        n, k = ids.shape
        # (``differentiable`` is the caller's word: inside a Function's forward the grad mode is always off, and the
        # inputs report requires_grad under torch.no_grad() as well)
        if row_ids is not None and token_of_row is None and differentiable:
            raise RuntimeError("row_ids without token_of_row cannot be differentiated")
        out = torch.empty((n, k), dtype=torch.float32, device=x.device)
        lse_out = lse if lse is not None else torch.empty(n, dtype=torch.float32, device=x.device)
        stride = x.stride(0) if x.size(0) > 1 else x.size(1)
        with ops._timed("topk_logprob_fwd"):
            check(lib.relax_amd_topk_logprob_fwd(_p(x), _code(x), n, x.size(1), stride, _p(row_ids), _p(ids), k,
                                                 float(inv_temperature), _p(lse), _p(out),
                                                 None if lse is not None else _p(lse_out), _stream()))
        ctx.save_for_backward(x, ids, lse_out, token_of_row)
        ctx.inv_temperature = float(inv_temperature)
        ctx.shape = logits.shape
        return out

    @staticmethod
    def backward(ctx, g):
        x, ids, lse, token_of_row = ctx.saved_tensors
        n, k = ids.shape
        d = torch.empty((x.size(0), x.size(1)), dtype=x.dtype, device=x.device)
        stride = x.stride(0) if x.size(0) > 1 else x.size(1)
        g = _f32(g).reshape(n, k).contiguous()
        with ops._timed("topk_logprob_bwd"):
            check(lib.relax_amd_topk_logprob_bwd(_p(x), _code(x), x.size(0), x.size(1), stride, _p(token_of_row),
                                                 _p(ids), k, ctx.inv_temperature, _p(lse), _p(g), _p(d), d.size(1),
                                                 _stream()))
        return d.view(ctx.shape), None, None, None, None, None, None


def compute_log_probs_on_topk_token_ids(logits: torch.Tensor, topk_token_ids: torch.Tensor, process_group=None,
                                        temperature: float = 1.0, lse: torch.Tensor | None = None) -> torch.Tensor:
    """``[S, K]`` log-probabilities of the given (global) vocabulary ids, opd_utils.py:1022-1094 on one rank: ids
    ``< 0`` are sentinels and yield ``-inf``.  ``lse`` (fp32 ``[S]``, the row log-sum-exps a log-prob forward already
    produced) turns the call into K loads per row; without it the kernel scans each row once.  Gradient flows to
    ``logits`` through both the gather and the log-sum-exp."""
    if process_group is not None and torch.distributed.is_initialized() and \
            torch.distributed.get_world_size(process_group) > 1:
        raise NotImplementedError("vocab-parallel top-K gather (tensor-parallel size > 1) is not supported")
    if logits.dim() != 2 or topk_token_ids.dim() != 2 or topk_token_ids.size(0) != logits.size(0):
        raise ValueError(f"expected logits [S, V] and ids [S, K], got {tuple(logits.shape)} and "
                         f"{tuple(topk_token_ids.shape)}")
    if logits.size(0) == 0:
        return logits.new_zeros((0, topk_token_ids.size(-1)))
    _need_gpu(logits)
    ids = topk_token_ids.to(device=logits.device, dtype=torch.long).contiguous()
    if ids.size(1) == 0:
        return torch.zeros((logits.size(0), 0), dtype=torch.float32, device=logits.device)
    if lse is not None:
        lse = _f32(lse).reshape(-1)
        if lse.numel() != logits.size(0):
            raise ValueError(f"lse has {lse.numel()} entries for {logits.size(0)} rows")
    return TopKLogProbs.apply(logits, ids, 1.0 / float(temperature), lse)


class _OpdKlTopk(torch.autograd.Function):
    @staticmethod
    def forward(ctx, s, t, mask, mode, norm, alpha, clamp):
        n, k = s.shape
        kl = torch.empty(n, dtype=torch.float32, device=s.device)
        has_clamp, cval = (0, 0.0) if clamp is None else (1, float(clamp))
        check(lib.relax_amd_opd_kl_topk_fwd(_p(s), _p(t), _p(mask), n, k, mode, norm, alpha, has_clamp, cval, _p(kl),
                                            _stream()))
        ctx.save_for_backward(s, t, mask)
        ctx.cfg = (mode, norm, alpha, has_clamp, cval)
        return kl

    @staticmethod
    def backward(ctx, g):
        s, t, mask = ctx.saved_tensors
        mode, norm, alpha, has_clamp, cval = ctx.cfg
        n, k = s.shape
        d = torch.empty_like(s)
        g = _f32(g).reshape(-1).contiguous()
        check(lib.relax_amd_opd_kl_topk_bwd(_p(s), _p(t), _p(mask), n, k, mode, norm, alpha, has_clamp, cval, _p(g),
                                            _p(d), _stream()))
        return d, None, None, None, None, None, None


def opd_topk_kernel_modes(kl_type: str, jsd_alpha: float, norm_mode: str):
    """``(kl mode, jsd alpha, norm mode)`` codes of the top-K KL kernels for the reference's option strings
    (opd_utils.py:1190-1228); raises as ``compute_opd_kl_topk`` does on unknown ones."""
    if kl_type not in OPD_KL_TYPES:
        raise ValueError(f"Unknown opd_kl_type: {kl_type}. Choose one of {OPD_KL_TYPES}.")
    if kl_type == "low_var_kl":
        mode, alpha = _lib.OPD_LOW_VAR, 0.0
    else:
        mode = _lib.OPD_JSD
        alpha = {"reverse_kl": 0.0, "forward_kl": 1.0}.get(kl_type, float(jsd_alpha))
        if not (0.0 <= alpha <= 1.0):
            raise ValueError(f"jsd_alpha must be in [0, 1], got {jsd_alpha}")
    if norm_mode not in _NORM_MODES:
        raise ValueError(f"Unknown opd_norm_mode: {norm_mode}. Choose one of {tuple(_NORM_MODES)}.")
    return mode, alpha, _NORM_MODES[norm_mode]


def compute_opd_kl_topk(student_topk_lp: torch.Tensor, teacher_topk_lp: torch.Tensor, kl_type: str = "reverse_kl",
                        jsd_alpha: float = 0.5, norm_mode: str = "tail", log_prob_min_clamp: float | None = None,
                        mask: torch.Tensor | None = None) -> torch.Tensor:
    """Per-token KL ``[R]`` (fp32) from ``[R, K]`` top-K log-probs, opd_utils.py:1190-1228: reverse / forward KL are
    the ``jsd_alpha`` = 0 / 1 ends of the JSD family, ``low_var_kl`` is summed element-wise over K.  ``mask`` (bool
    ``[R, K]``, True = valid) is the union path's padding mask.  Differentiable w.r.t. the student log-probs."""
    mode, alpha, norm = opd_topk_kernel_modes(kl_type, jsd_alpha, norm_mode)
    if student_topk_lp.dim() != 2 or student_topk_lp.shape != teacher_topk_lp.shape:
        raise ValueError(f"expected matching [R, K] inputs, got {tuple(student_topk_lp.shape)} and "
                         f"{tuple(teacher_topk_lp.shape)}")
    _need_gpu(student_topk_lp)
    dev = student_topk_lp.device
    s = student_topk_lp.to(torch.float32).contiguous()
    t = teacher_topk_lp.detach().to(device=dev, dtype=torch.float32).contiguous()
    if mask is not None:
        if mask.shape != s.shape:
            raise ValueError(f"mask {tuple(mask.shape)} does not match the inputs {tuple(s.shape)}")
        mask = mask.to(device=dev, dtype=torch.uint8).contiguous()
    if s.size(0) == 0:
        return s.sum(dim=-1)
    return _OpdKlTopk.apply(s, t, mask, mode, norm, alpha, log_prob_min_clamp)


def compute_opd_kl(student_log_probs, teacher_log_probs, kl_type: str = "reverse_kl", jsd_alpha: float = 0.5,
                   norm_mode: str = "tail", log_prob_min_clamp: float | None = None, mask=None):
    """Per-token OPD signal (opd_utils.py:1097-1187).  1-D sampled-token inputs: ``reverse_kl`` (k1) and
    ``low_var_kl`` (k3), evaluated by the policy-loss kernel's KL estimators.  2-D ``[R, K]`` inputs: ``jsd`` and
    ``low_var_kl`` through the top-K kernel."""
    from .ppo_utils import compute_approx_kl

    if student_log_probs.dim() == 2:
        if kl_type in ("jsd", "low_var_kl"):
            return compute_opd_kl_topk(student_log_probs, teacher_log_probs, kl_type, jsd_alpha, norm_mode,
                                       log_prob_min_clamp, mask)
        if kl_type != "reverse_kl":
            raise ValueError(f"Unknown opd_kl_type: {kl_type}. Choose one of {OPD_KL_TYPES}.")
        # opd_utils.py:1126-1138: for [R, K] inputs "reverse_kl" is the element-wise log-ratio itself (padding of a
        # union mask gives -inf - -inf there, as in the reference); callers that want the summed KL use
        # compute_opd_kl_topk
        s, t = student_log_probs.float(), teacher_log_probs.float()
        if log_prob_min_clamp is not None:
            s, t = s.clamp_min(log_prob_min_clamp), t.clamp_min(log_prob_min_clamp)
        if mask is not None:
            s, t = s.masked_fill(~mask, float("-inf")), t.masked_fill(~mask, float("-inf"))
        return s - t
    s, t = student_log_probs, teacher_log_probs
    if log_prob_min_clamp is not None:
        s, t = s.clamp_min(log_prob_min_clamp), t.clamp_min(log_prob_min_clamp)
    if kl_type == "reverse_kl":
        return compute_approx_kl(s, t, "k1")
    if kl_type == "low_var_kl":
        return compute_approx_kl(s, t, "k3")
    raise ValueError(f"Unknown opd_kl_type: {kl_type}. Choose one of {OPD_KL_TYPES}.")


class _TokenMean(torch.autograd.Function):
    @staticmethod
    def forward(ctx, values, mask, cu):
        num = ops.segment_sum(mask, cu, values=values).sum()
        den = torch.clamp_min(ops.segment_sum(mask, cu).sum(), 1)
        ctx.save_for_backward(mask, den)
        return (num / den).to(torch.float32)

    @staticmethod
    def backward(ctx, g):
        mask, den = ctx.saved_tensors
        return (mask * (g / den)).to(torch.float32), None, None


def reduce_opd_loss(batch: dict, values: torch.Tensor) -> torch.Tensor:
    """``sum(values * mask) / clamp_min(sum mask, 1)`` over the whole micro-batch."""
    dev = values.device
    mask = torch.cat([m.reshape(-1) for m in batch["loss_masks"]]).to(device=dev, dtype=torch.float32)
    return _TokenMean.apply(values.to(torch.float32), mask, _cu(batch["response_lengths"], dev))


class _FusedOpdLoss(torch.autograd.Function):
    """student logits [N, V] -> (masked token-mean reverse KL, per-token KL), one launch: the gradient of the token
    mean w.r.t. each token's KL (mask / clamp_min(sum mask, 1)) is known before the forward, so the kernel writes the
    student gradient for an upstream gradient of 1 while the rows are still in cache; the backward multiplies by the
    actual upstream gradient over the assumed one (``batch["relax_amd_grad_scale"]``, default 1) on the device: a
    no-op kernel when they agree."""

    @staticmethod
    def forward(ctx, student, teacher, mask, assumed_scale=1.0):
        den = torch.clamp_min(mask.sum(), 1)
        g = mask / den
        kl, _ls, _lt, d = ops.reverse_kl_step_fused(student, teacher, g if assumed_scale == 1.0 else g * assumed_scale)
        ctx.d = d
        ctx.shape = student.shape
        ctx.assumed_scale = float(assumed_scale)
        ctx.mark_non_differentiable(kl)
        return (kl * mask).sum() / den, kl

    @staticmethod
    def backward(ctx, g_loss, _g_kl):
        d = ctx.d
        if d is None:
            raise RuntimeError("the fused OPD loss holds its gradient once: backward cannot run twice")
        ctx.d = None
        factor = g_loss.reshape(1).to(torch.float32)
        if ctx.assumed_scale != 1.0:
            factor = factor / ctx.assumed_scale
        ops.scale_rows_inplace(d, factor.contiguous())
        return d.view(ctx.shape), None, None, None


def opd_loss_full_vocab(batch: dict, student_logits: torch.Tensor, teacher_logits: torch.Tensor):
    """``reduce_opd_loss(batch, compute_opd_kl_full_vocab(student, teacher))`` in a single kernel launch
    (opd_utils.py:1165-1169 + :1355-1365).  Returns ``(loss, per_token_kl)``; differentiable w.r.t. the student."""
    dev = student_logits.device
    mask = torch.cat([m.reshape(-1) for m in batch["loss_masks"]]).to(device=dev, dtype=torch.float32)
    rows = student_logits.reshape(-1, student_logits.size(-1))
    if mask.numel() != rows.size(0):
        raise ValueError(f"loss masks cover {mask.numel()} tokens, logits have {rows.size(0)} rows")
    if not (torch.is_grad_enabled() and student_logits.requires_grad):
        kl = compute_opd_kl_full_vocab(student_logits, teacher_logits)
        return reduce_opd_loss(batch, kl), kl
    from .loss import expected_grad_scale

    return _FusedOpdLoss.apply(student_logits, teacher_logits.detach(), mask, expected_grad_scale(batch))


def resolve_opd_gather_topk_token_ids(args, batch):
    """opd_utils.py:999-1003: the ids whose log-probs the forward must gather, for the top-K token selections."""
    if getattr(args, "opd_token_selection", None) in ("student_topk", "teacher_topk", "union"):
        return batch.get("opd_topk_token_ids", None)
    return None


def compute_policy_opd_loss(*, args, batch, log_probs, old_log_probs, log_probs_and_entropy):
    """``opd_loss_coef`` times the masked token mean of the per-token distillation signal (opd_utils.py:1368-1455):
    top-K (per sample, with the union path's length mask) or sampled-token, after the optional per-token clip and
    importance-ratio clip.  Returns ``(loss | None, metrics)``; differentiable through ``log_probs`` and the gathered
    ``topk_log_probs``."""
    coef = float(getattr(args, "opd_loss_coef", 0.0) or 0.0)
    if coef == 0.0:
        return None, {}
    kl_type = args.opd_kl_type
    alpha = float(args.opd_jsd_alpha)
    norm = getattr(args, "opd_norm_mode", "tail")
    clamp = getattr(args, "opd_log_prob_min_clamp", None)
    selection = args.opd_token_selection
    dev = log_probs.device
    if selection in ("student_topk", "teacher_topk", "union"):
        student = log_probs_and_entropy.get("topk_log_probs")
        teacher = batch.get("opd_topk_teacher_log_probs")
        if not (student and teacher):
            return None, {}
        ksz = batch.get("opd_topk_ksz") if selection == "union" else None
        parts = []
        for i, s_lp in enumerate(student):
            t_lp = teacher[i].to(device=dev).detach()
            mask = None
            if ksz is not None and i < len(ksz) and ksz[i] is not None:
                mask = torch.arange(t_lp.size(-1), device=dev).unsqueeze(0) < ksz[i].to(dev).unsqueeze(1)
            parts.append(compute_opd_kl_topk(s_lp, t_lp, kl_type, alpha, norm, clamp, mask))
        per_token = torch.cat(parts, dim=0).to(log_probs.dtype)
    else:
        if batch.get("teacher_log_probs") is None:
            return None, {}
        teacher = torch.cat(batch["teacher_log_probs"], dim=0).to(device=dev, dtype=log_probs.dtype).detach()
        per_token = compute_opd_kl(log_probs, teacher, kl_type, alpha, norm, clamp).to(log_probs.dtype)
    return finish_policy_opd_loss(args, batch, per_token, log_probs, old_log_probs)


def finish_policy_opd_loss(args, batch, per_token, log_probs, old_log_probs):
    """The tail of ``compute_policy_opd_loss`` on the per-token signal ``[N]``: per-token clip, importance-ratio clip
    (ratio detached), ``opd_loss_coef`` times the masked token mean, and the two clip-fraction metrics."""
    reported = {}
    tau = getattr(args, "opd_per_token_clip", None)
    if tau is not None:
        before = per_token
        per_token = torch.clamp(per_token, max=float(tau))
        with torch.no_grad():
            reported["opd_per_token_clip_frac"] = (before > float(tau)).float().mean().clone().detach()
    clip = getattr(args, "opd_is_clip", None)
    if clip is not None:
        ratio = torch.exp(log_probs.detach() - old_log_probs.detach())
        per_token = per_token * torch.clamp(ratio, max=float(clip)).to(per_token.dtype)
        with torch.no_grad():
            reported["opd_is_clip_frac"] = (ratio > float(clip)).float().mean().clone().detach()
    return float(args.opd_loss_coef) * reduce_opd_loss(batch, per_token), reported


def apply_opd_to_advantages(args, rollout_data, advantages: list) -> None:
    """``advantages[i] -= opd_kl_coef * per_token_signal`` in place (opd_utils.py:1275-1351): the top-K signal from the
    rollout's stored student / teacher top-K log-probs (with the union path's length mask and the per-token clip), or
    the sampled-token signal from ``rollout_log_probs`` / ``teacher_log_probs``."""
    if args.opd_kl_coef == 0.0:
        return
    kl_type = args.opd_kl_type
    alpha = float(args.opd_jsd_alpha)
    norm = getattr(args, "opd_norm_mode", "tail")
    clamp = getattr(args, "opd_log_prob_min_clamp", None)
    selection = args.opd_token_selection
    if selection in ("student_topk", "teacher_topk", "union"):
        student = rollout_data.get("opd_topk_student_log_probs")
        teacher = rollout_data.get("opd_topk_teacher_log_probs")
        if student is None or teacher is None:
            return
        ksz = rollout_data.get("opd_topk_ksz") if selection == "union" else None
        tau = getattr(args, "opd_per_token_clip", None)
        for i, adv in enumerate(advantages):
            dev = adv.device
            s_lp = student[i].to(dev) if i < len(student) and isinstance(student[i], torch.Tensor) else None
            t_lp = teacher[i].to(dev) if i < len(teacher) and isinstance(teacher[i], torch.Tensor) else None
            if s_lp is None or t_lp is None or s_lp.numel() == 0 or s_lp.shape != t_lp.shape:
                raise ValueError(f"OPD per-token signal: token_selection={selection} but the required arms are missing.")
            mask = None
            if ksz is not None and i < len(ksz) and ksz[i] is not None:
                mask = torch.arange(t_lp.size(-1), device=dev).unsqueeze(0) < ksz[i].to(dev).unsqueeze(1)
            term = compute_opd_kl_topk(s_lp, t_lp, kl_type, alpha, norm, clamp, mask).to(s_lp.dtype)
            if tau is not None:
                term = torch.clamp(term, max=float(tau))
            advantages[i] = adv - args.opd_kl_coef * term.detach()
        return
    student = rollout_data.get("rollout_log_probs")
    teacher = rollout_data.get("teacher_log_probs")
    if student is None or teacher is None:
        return
    for i, adv in enumerate(advantages):
        term = compute_opd_kl(student[i], teacher[i].to(student[i].device), kl_type, alpha, norm, clamp)
        advantages[i] = adv - args.opd_kl_coef * term.detach().to(student[i].dtype)
