"""Oracle: target-token log-prob + full-vocab entropy and their backward.

Test infrastructure only (see ``oracle/__init__.py``).

Follows relax/utils/training/ppo_utils.py:480-629 (the single-rank behaviour of
``_VocabParallelLogProbEntropy``) and :1192-1243 (the row-chunk driver).  The
op ORDER of the reference is kept (upcast, row max, shift, gather, exp, sum,
divide, sum(p*x)) so fp32 results agree with it to rounding; the code layout is
this build's own.
"""

from __future__ import annotations

import torch


def softmax_pieces(x32: torch.Tensor):
    """ppo_utils.py:503-522 -- max, shift, exp, sum, divide, in that order.

    Returns (shifted logits, row max [N,1], sum exp [N,1], softmax [N,V]).
    """
    row_max = x32.max(dim=-1, keepdim=True).values
    shifted = x32 - row_max
    ex = shifted.exp()
    denom = ex.sum(dim=-1, keepdim=True)
    return shifted, row_max, denom, ex / denom


def forward_values(logits: torch.Tensor, tokens: torch.Tensor, keep_mask: torch.Tensor | None, with_entropy: bool):
    """Forward arithmetic of ppo_utils.py:481-589 on one rank (vocab_start = 0).

    logits [N,V] any float dtype, tokens [N] int64, keep_mask [N,V] bool or None.
    Returns dict with lp [N,1] fp32, entropy [N] fp32 (or empty), and the saved
    pieces the explicit backward needs.
    """
    x = logits.float()
    n, v = x.shape
    rows = torch.arange(n, device=x.device)
    entropy = x.new_zeros((0,))
    ent_softmax = None
    spx = None
    if keep_mask is None:
        shifted, row_max, denom, p = softmax_pieces(x)
        picked = shifted[rows, tokens]
        if with_entropy:
            ent_softmax = p
            spx = (p * x).sum(dim=-1, keepdim=True)  # :528-532
            entropy = (row_max + denom.log() - spx).squeeze(-1)  # :542
    else:
        if with_entropy:
            _, e_max, e_denom, ent_softmax = softmax_pieces(x)
            spx = (ent_softmax * x).sum(dim=-1, keepdim=True)
            entropy = (e_max + e_denom.log() - spx).squeeze(-1)  # :551
        # :554-564 -- softmax restricted to kept ids, target always kept
        restricted = x.masked_fill(~keep_mask, float("-inf"))
        restricted[rows, tokens] = x[rows, tokens]
        shifted, _, denom, p = softmax_pieces(restricted)
        picked = shifted[rows, tokens]
    lp = picked.unsqueeze(-1) - denom.log()  # :566-568
    return {"lp": lp, "entropy": entropy, "p_lp": p, "p_ent": ent_softmax, "spx": spx, "x": x}


def backward_values(saved: dict, tokens: torch.Tensor, g_lp: torch.Tensor, g_ent: torch.Tensor | None):
    """Explicit gradient of ppo_utils.py:591-629.

    dx = g_lp * (onehot(tok) - p_lp) + g_ent * p_ent * (sum_v p_ent*x - x)
    """
    p = saved["p_lp"]
    n = p.shape[0]
    rows = torch.arange(n, device=p.device)
    grad = -p.clone()
    grad[rows, tokens] += 1.0
    grad = grad * g_lp.reshape(-1, 1)
    if g_ent is not None and saved["p_ent"] is not None and g_ent.numel() > 0:
        grad = grad + (saved["spx"] - saved["x"]) * saved["p_ent"] * g_ent.reshape(-1, 1)
    return grad


class _LogProbEntropy(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits, tokens, keep_mask, with_entropy, with_entropy_grad):
        with_entropy_grad = bool(with_entropy and with_entropy_grad)
        saved = forward_values(logits, tokens, keep_mask, with_entropy)
        ctx.saved = saved if with_entropy_grad else {**saved, "p_ent": None, "spx": None, "x": None}
        ctx.tokens = tokens
        ctx.in_dtype = logits.dtype
        ctx.with_entropy_grad = with_entropy_grad
        if not with_entropy_grad:
            ctx.mark_non_differentiable(saved["entropy"])  # :570-571
        return saved["lp"], saved["entropy"]

    @staticmethod
    def backward(ctx, g_lp, g_ent):
        if g_lp is None:
            raise RuntimeError("expected a materialized grad_log_prob")  # :604-608
        g = backward_values(ctx.saved, ctx.tokens, g_lp, g_ent if ctx.with_entropy_grad else None)
        return g.to(ctx.in_dtype), None, None, None, None


def calculate_log_probs_and_entropy(
    logits: torch.Tensor,
    tokens: torch.Tensor,
    tp_group=None,
    with_entropy: bool = False,
    chunk_size: int = -1,
    log_prob_keep_mask: torch.Tensor | None = None,
    with_entropy_grad: bool = True,
):
    """Row-chunk driver, ppo_utils.py:1192-1243.  Returns (lp [N,1], entropy [N] | None)."""
    logits = logits.contiguous()
    if logits.size(0) == 0:
        return logits.new_zeros((0,)), (logits.new_zeros((0,)) if with_entropy else None)
    if chunk_size > 0:
        pieces = (logits.size(0) - 1) // chunk_size + 1
        l_parts = logits.chunk(pieces, dim=0)
        t_parts = tokens.chunk(pieces, dim=0)
        m_parts = log_prob_keep_mask.chunk(pieces, dim=0) if log_prob_keep_mask is not None else [None] * pieces
    else:
        l_parts, t_parts, m_parts = [logits], [tokens], [log_prob_keep_mask]
    lps, ents = [], []
    for lg, tk, mk in zip(l_parts, t_parts, m_parts, strict=True):
        lp, ent = _LogProbEntropy.apply(lg, tk, mk, with_entropy, with_entropy_grad)
        lps.append(lp)
        if with_entropy:
            ents.append(ent)
    lp = torch.cat(lps, dim=0) if len(lps) > 1 else lps[0]
    ent = None
    if with_entropy:
        ent = torch.cat(ents, dim=0) if len(ents) > 1 else ents[0]
    return lp, ent
