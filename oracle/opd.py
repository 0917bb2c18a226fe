"""Oracle: on-policy-distillation KL signals.

Test infrastructure only.  Follows relax/utils/opd/opd_utils.py:1097-1228 (per-token KL on sampled-token or
[R,K] log-probs) and :1355-1365 (token-mean reduction).  The full-vocab reverse KL named by the benchmark is
the K = V case of the ``jsd_alpha == 0`` branch (:1165-1169) fed with complete ``log_softmax`` rows.
"""

from __future__ import annotations

import torch


def _with_tail(lp):
    # :1146-1149 -- append log(1 - sum p) with logsumexp clamped to <= -1e-7
    ls = torch.logsumexp(lp, dim=-1, keepdim=True).clamp(max=-1e-7)
    return torch.cat([lp, torch.log(-torch.expm1(ls))], dim=-1)


def opd_kl(s_lp, t_lp, kl_type="reverse_kl", jsd_alpha=0.5, norm_mode="tail", min_clamp=None):
    """opd_utils.py:1097-1187 without the union-path padding mask."""
    s, t = s_lp.float(), t_lp.float()
    if min_clamp is not None:
        s, t = s.clamp_min(min_clamp), t.clamp_min(min_clamp)
    d = s - t
    if kl_type == "reverse_kl":
        return d
    if kl_type == "low_var_kl":
        per = torch.exp(-d) - 1.0 + d
        return per.sum(dim=-1) if per.dim() > 1 else per
    if kl_type != "jsd":
        raise ValueError(f"Unknown opd_kl_type: {kl_type}.")
    if not (0.0 <= jsd_alpha <= 1.0):
        raise ValueError(f"jsd_alpha must be in [0, 1], got {jsd_alpha}")
    if norm_mode == "tail":
        s, t = _with_tail(s), _with_tail(t)
    elif norm_mode == "norm":
        s = s - torch.logsumexp(s, dim=-1, keepdim=True)
        t = t - torch.logsumexp(t, dim=-1, keepdim=True)
    if jsd_alpha == 0.0:
        return (s.exp() * (s - t)).sum(dim=-1)
    if jsd_alpha == 1.0:
        return (t.exp() * (t - s)).sum(dim=-1)
    l1 = torch.log(torch.tensor(1.0 - jsd_alpha, dtype=s.dtype))
    la = torch.log(torch.tensor(jsd_alpha, dtype=s.dtype))
    mix = torch.logsumexp(torch.stack([s + l1, t + la]), dim=0)
    return (1.0 - jsd_alpha) * (s.exp() * (s - mix)).sum(-1) + jsd_alpha * (t.exp() * (t - mix)).sum(-1)


def opd_kl_topk(s_lp, t_lp, kl_type="reverse_kl", jsd_alpha=0.5, norm_mode="tail", min_clamp=None):
    """opd_utils.py:1190-1228: reverse/forward KL are the alpha = 0 / 1 ends of the JSD family."""
    if kl_type in ("reverse_kl", "forward_kl", "jsd"):
        alpha = {"reverse_kl": 0.0, "forward_kl": 1.0}.get(kl_type, float(jsd_alpha))
        return opd_kl(s_lp, t_lp, "jsd", alpha, norm_mode, min_clamp)
    per = opd_kl(s_lp, t_lp, kl_type, min_clamp=min_clamp)
    return per.sum(dim=-1) if per.dim() > 1 else per


def full_vocab_reverse_kl(student_logits, teacher_logits, norm_mode="tail"):
    """K = V: per-token sum_v p_s (log p_s - log p_t) through the reference's top-K code path."""
    s = torch.log_softmax(student_logits.float(), dim=-1)
    t = torch.log_softmax(teacher_logits.float(), dim=-1)
    return opd_kl_topk(s, t, "reverse_kl", norm_mode=norm_mode)


def reduce_token_mean(values, response_lengths, masks):
    """opd_utils.py:1355-1365."""
    parts = [c * m.to(c.dtype) for c, m in zip(torch.split(values, response_lengths, dim=0), masks, strict=False)]
    den = sum(m.to(values.dtype).sum() for m in masks)
    return torch.cat(parts, dim=0).sum() / torch.clamp_min(den, 1)
