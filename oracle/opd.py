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


def opd_kl(s_lp, t_lp, kl_type="reverse_kl", jsd_alpha=0.5, norm_mode="tail", min_clamp=None, mask=None):
    """opd_utils.py:1097-1187.  ``mask`` (bool [R, K], True = valid) is the union path's padding mask (:1121-1127):
    padded entries are set to -inf after the clamp, and the summed terms are cut back to the first K columns and
    zeroed at the padding -- which also drops the tail bin (:1158-1186)."""
    s, t = s_lp.float(), t_lp.float()
    if min_clamp is not None:
        s, t = s.clamp_min(min_clamp), t.clamp_min(min_clamp)
    if mask is not None:
        s, t = s.masked_fill(~mask, float("-inf")), t.masked_fill(~mask, float("-inf"))
    d = s - t
    if kl_type == "reverse_kl":
        return d
    if kl_type == "low_var_kl":
        per = torch.exp(-d) - 1.0 + d
        if mask is not None:
            per = per.masked_fill(~mask, 0.0)
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

    def total(terms):
        if mask is not None:
            terms = terms[..., : mask.size(-1)].masked_fill(~mask, 0.0)
        return terms.sum(dim=-1)

    if jsd_alpha == 0.0:
        return total(s.exp() * (s - t))
    if jsd_alpha == 1.0:
        return total(t.exp() * (t - s))
    l1 = torch.log(torch.tensor(1.0 - jsd_alpha, dtype=s.dtype))
    la = torch.log(torch.tensor(jsd_alpha, dtype=s.dtype))
    mix = torch.logsumexp(torch.stack([s + l1, t + la]), dim=0)
    return (1.0 - jsd_alpha) * total(s.exp() * (s - mix)) + jsd_alpha * total(t.exp() * (t - mix))


def opd_kl_topk(s_lp, t_lp, kl_type="reverse_kl", jsd_alpha=0.5, norm_mode="tail", min_clamp=None, mask=None):
    """opd_utils.py:1190-1228: reverse/forward KL are the alpha = 0 / 1 ends of the JSD family."""
    if kl_type in ("reverse_kl", "forward_kl", "jsd"):
        alpha = {"reverse_kl": 0.0, "forward_kl": 1.0}.get(kl_type, float(jsd_alpha))
        return opd_kl(s_lp, t_lp, "jsd", alpha, norm_mode, min_clamp, mask)
    per = opd_kl(s_lp, t_lp, kl_type, min_clamp=min_clamp, mask=mask)
    return per.sum(dim=-1) if per.dim() > 1 else per


def log_probs_on_topk_ids(logits, ids):
    """compute_log_probs_on_topk_token_ids (opd_utils.py:1022-1094) on one rank: ``logits[ids] - logsumexp(logits)``
    per row; ids < 0 are sentinels and give -inf, ids >= V read as logit 0 (the reference's out-of-slice fill)."""
    if logits.size(0) == 0:
        return logits.new_zeros((0, ids.size(-1)))
    x = logits
    lse = torch.logsumexp(x.float(), dim=-1, keepdim=True).to(x.dtype)
    ids = ids.to(torch.long)
    safe = ids.clamp(min=0)
    inside = safe < x.size(-1)
    got = torch.gather(x, -1, safe.clamp(max=x.size(-1) - 1)).masked_fill(~inside, 0.0)
    return (got - lse).masked_fill(ids < 0, float("-inf"))


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


def policy_opd_loss(args, batch, log_probs, old_log_probs, topk_log_probs):
    """compute_policy_opd_loss, opd_utils.py:1368-1455: ``opd_loss_coef`` times the masked token mean of the per-token
    distillation signal -- top-K (per sample, with the union path's length mask) or sampled-token -- after the
    optional per-token clip and importance-ratio clip.  Returns (loss | None, metrics)."""
    coef = float(getattr(args, "opd_loss_coef", 0.0))
    if coef == 0.0:
        return None, {}
    kl_type, alpha = args.opd_kl_type, float(args.opd_jsd_alpha)
    norm = getattr(args, "opd_norm_mode", "tail")
    clamp = getattr(args, "opd_log_prob_min_clamp", None)
    sel = args.opd_token_selection
    teacher_topk = batch.get("opd_topk_teacher_log_probs")
    if sel in ("student_topk", "teacher_topk", "union"):
        if not (topk_log_probs and teacher_topk):
            return None, {}
        ksz = batch.get("opd_topk_ksz") if sel == "union" else None
        parts = []
        for i, s_lp in enumerate(topk_log_probs):
            t_lp = teacher_topk[i].detach()
            mask = None
            if ksz is not None and i < len(ksz) and ksz[i] is not None:
                mask = torch.arange(t_lp.size(-1)).unsqueeze(0) < ksz[i].unsqueeze(1)
            parts.append(opd_kl_topk(s_lp, t_lp, kl_type, alpha, norm, clamp, mask))
        per_token = torch.cat(parts, dim=0).to(log_probs.dtype)
    else:
        if batch.get("teacher_log_probs") is None:
            return None, {}
        teacher = torch.cat(batch["teacher_log_probs"], dim=0).to(log_probs.dtype).detach()
        per_token = opd_kl(log_probs, teacher, kl_type, alpha, norm, clamp).to(log_probs.dtype)
    metrics = {}
    tau = getattr(args, "opd_per_token_clip", None)
    if tau is not None:
        before = per_token
        per_token = torch.clamp(per_token, max=float(tau))
        metrics["opd_per_token_clip_frac"] = (before > float(tau)).float().mean().detach()
    clip = getattr(args, "opd_is_clip", None)
    if clip is not None:
        ratio = torch.exp(log_probs.detach() - old_log_probs.detach())
        per_token = per_token * torch.clamp(ratio, max=float(clip)).to(per_token.dtype)
        metrics["opd_is_clip_frac"] = (ratio > float(clip)).float().mean().detach()
    return coef * reduce_token_mean(per_token, batch["response_lengths"], batch["loss_masks"]), metrics


def apply_to_advantages(args, rollout_data, advantages: list) -> None:
    """apply_opd_to_advantages, opd_utils.py:1275-1351: ``advantages[i] -= opd_kl_coef * signal_i`` in place."""
    if args.opd_kl_coef == 0.0:
        return
    kl_type, alpha = args.opd_kl_type, float(args.opd_jsd_alpha)
    norm = getattr(args, "opd_norm_mode", "tail")
    clamp = getattr(args, "opd_log_prob_min_clamp", None)
    sel = args.opd_token_selection
    if sel in ("student_topk", "teacher_topk", "union"):
        student, teacher = rollout_data.get("opd_topk_student_log_probs"), rollout_data.get("opd_topk_teacher_log_probs")
        if student is None or teacher is None:
            return
        ksz = rollout_data.get("opd_topk_ksz") if sel == "union" else None
        for i, adv in enumerate(advantages):
            mask = None
            if ksz is not None and ksz[i] is not None:
                mask = torch.arange(teacher[i].size(-1)).unsqueeze(0) < ksz[i].unsqueeze(1)
            term = opd_kl_topk(student[i], teacher[i], kl_type, alpha, norm, clamp, mask).to(student[i].dtype)
            tau = getattr(args, "opd_per_token_clip", None)
            if tau is not None:
                term = torch.clamp(term, max=float(tau))
            advantages[i] = adv - args.opd_kl_coef * term.detach()
        return
    student, teacher = rollout_data.get("rollout_log_probs"), rollout_data.get("teacher_log_probs")
    if student is None or teacher is None:
        return
    for i, adv in enumerate(advantages):
        term = opd_kl(student[i], teacher[i], kl_type, alpha, norm, clamp).to(student[i].dtype)
        advantages[i] = adv - args.opd_kl_coef * term.detach()
