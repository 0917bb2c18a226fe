"""SFT perplexity evaluation: the forward-only callback and the final aggregation.

Counterpart of relax/engine/sft/eval/ppl.py: ``compute_sft_eval_step`` has the ``f(logits, *, args, ...)`` signature the
forward-only harness calls per micro-batch (relax/backends/megatron/model.py:838-852) and returns the masked sum of
negative log-probs and the token count as one-element tensors; ``compute_ppl_metrics`` turns the reduced totals into
``eval/loss`` / ``eval/ppl`` / ``eval/num_tokens``.  Context parallel size 1.
"""

from __future__ import annotations

import math

import torch


def compute_sft_eval_step(logits: torch.Tensor, *, args, unconcat_tokens, total_lengths, response_lengths,
                          with_entropy: bool = False, loss_masks=None, lm_head_forward=None, max_seq_lens=None, **_):
    """``(empty tensor, {"sum_neg_log_prob": [fp32 [1]], "num_tokens": [int64 [1]]})`` (ppl.py:24-92).  ``logits`` may
    be hidden states when ``lm_head_forward`` is given, as for ``get_log_probs_and_entropy``."""
    from .cp_utils import get_sum_of_sample_mean
    from .loss import get_log_probs_and_entropy

    assert loss_masks is not None, "compute_sft_eval_step requires loss_masks (passed by forward_step)."
    with torch.no_grad():
        _, res = get_log_probs_and_entropy(logits, args=args, unconcat_tokens=unconcat_tokens,
                                           total_lengths=total_lengths, response_lengths=response_lengths,
                                           with_entropy=False, lm_head_forward=lm_head_forward,
                                           max_seq_lens=max_seq_lens)
        flat = torch.cat(res["log_probs"], dim=0)
        token_sum = get_sum_of_sample_mean(total_lengths, response_lengths, loss_masks, calculate_per_token_loss=True)
        sum_neg_lp = -token_sum(flat)
        num_tokens = token_sum(torch.ones_like(flat))
    return torch.empty((0,), device=flat.device), {
        "sum_neg_log_prob": [sum_neg_lp.reshape(1).to(torch.float32)],
        "num_tokens": [num_tokens.reshape(1).to(torch.long)],
    }


def compute_ppl_metrics(total_neg_log_prob: float, total_tokens: int) -> dict:
    """ppl.py:95-108: mean negative log-likelihood per token and its exponential; all zeros for an empty evaluation."""
    if total_tokens == 0:
        return {"eval/loss": 0.0, "eval/ppl": 0.0, "eval/num_tokens": 0}
    loss = total_neg_log_prob / total_tokens
    return {"eval/loss": loss, "eval/ppl": math.exp(loss), "eval/num_tokens": total_tokens}
