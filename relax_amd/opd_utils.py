"""On-policy-distillation KL on full-vocabulary logits (gfx950 kernels) and the reference's token-mean reduction.

``compute_opd_kl_full_vocab`` is the K = vocab case of ``compute_opd_kl``'s ``jsd_alpha == 0`` branch
(relax/utils/opd/opd_utils.py:1097-1228) evaluated straight from logits, so the [N, V] log-softmax tensors of the
student and the teacher are never materialised.  ``reduce_opd_loss`` follows :1355-1365.
"""

from __future__ import annotations

import torch

from . import ops
from .cp_utils import _cu


def compute_opd_kl_full_vocab(student_logits: torch.Tensor, teacher_logits: torch.Tensor) -> torch.Tensor:
    """Per-token reverse KL(student || teacher) over the whole vocabulary, fp32 [N]; differentiable w.r.t. the
    student logits (the teacher is treated as detached, as the reference detaches teacher log-probs)."""
    return ops.ReverseKL.apply(student_logits, teacher_logits.detach())


def compute_opd_kl(student_log_probs, teacher_log_probs, kl_type: str = "reverse_kl", **_):
    """Sampled-token (1-D) signals of opd_utils.py:1133-1141, evaluated by the policy-loss kernel's KL estimators."""
    from .ppo_utils import compute_approx_kl

    if student_log_probs.dim() != 1:
        raise NotImplementedError("[R, K] top-K inputs: use compute_opd_kl_full_vocab on logits for K = vocab")
    if kl_type == "reverse_kl":
        return compute_approx_kl(student_log_probs, teacher_log_probs, "k1")
    if kl_type == "low_var_kl":
        return compute_approx_kl(student_log_probs, teacher_log_probs, "k3")
    raise ValueError(f"Unknown opd_kl_type: {kl_type}.")


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
    actual upstream gradient on the device (a no-op kernel when it is exactly 1)."""

    @staticmethod
    def forward(ctx, student, teacher, mask):
        den = torch.clamp_min(mask.sum(), 1)
        g = mask / den
        kl, _ls, _lt, d = ops.reverse_kl_step_fused(student, teacher, g)
        ctx.d = d
        ctx.shape = student.shape
        ctx.mark_non_differentiable(kl)
        return (kl * mask).sum() / den, kl

    @staticmethod
    def backward(ctx, g_loss, _g_kl):
        d = ctx.d
        if d is None:
            raise RuntimeError("the fused OPD loss holds its gradient once: backward cannot run twice")
        ctx.d = None
        ops.scale_rows_inplace(d, g_loss.reshape(1).to(torch.float32).contiguous())
        return d.view(ctx.shape), None, None


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
    return _FusedOpdLoss.apply(student_logits, teacher_logits.detach(), mask)
