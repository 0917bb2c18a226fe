"""Oracle: masked reducers and token counts at context-parallel size 1.

Test infrastructure only.  Follows relax/backends/megatron/cp_utils.py:125-162
(the reducers) and :209-285 (token count incl. the per-sample clamp_min(1)).
"""

from __future__ import annotations

import torch


def sample_denominators(masks: list, sample_denoms=None):
    """cp_utils.py:138-142: per-sample sum of the mask, or the supplied per-sample denominators."""
    if sample_denoms is None:
        return torch.stack([m.sum() for m in masks])
    return torch.as_tensor(sample_denoms, device=masks[0].device)


def make_reducer(response_lengths: list, masks: list, per_token: bool = False, sample_denoms=None):
    """cp_utils.py:144-162,206.  per_token=False -> sum of per-sample masked means; True -> masked token sum."""
    if per_token:

        def token_sum(x):
            return sum((xi * mi).sum() for xi, mi in zip(x.split(response_lengths, dim=0), masks, strict=False))

        return token_sum
    den = sample_denominators(masks, sample_denoms)

    def sample_mean_sum(x):
        return sum(
            (xi * mi).sum() / torch.clamp_min(d, 1)
            for xi, mi, d in zip(x.split(response_lengths, dim=0), masks, den, strict=False)
        )

    return sample_mean_sum


def num_tokens(masks: list) -> torch.Tensor:
    """cp_utils.py:222,283-285: sum_i clamp_min(sum(mask_i), 1) -- a fully masked sample counts as one."""
    return torch.clamp_min(torch.stack([m.sum() for m in masks]), 1).sum()


def seq_mean_token_sum(response_lengths: list, masks: list):
    """sum_i sum_t x*m / B: each sequence's masked token sum, averaged over the B sequences.  The reference only has
    the plug-in point for such a reducer (loss.py:1062-1072) and no implementation, so this definition is the
    contract; tests/test_oracle_losses.py pins it by a token loop."""
    b = len(response_lengths)

    def red(x):
        return sum((xi * mi).sum() for xi, mi in zip(x.split(response_lengths, dim=0), masks, strict=False)) / b

    return red


def token_mean(response_lengths: list, masks: list):
    """relax/utils/opd/opd_utils.py:1355-1365: sum(x*m) / clamp_min(sum m, 1) over the whole micro-batch."""

    def red(x):
        num = torch.cat([c * m.to(c.dtype) for c, m in zip(x.split(response_lengths, dim=0), masks, strict=False)]).sum()
        den = sum(m.to(x.dtype).sum() for m in masks)
        return num / torch.clamp_min(den, 1)

    return red
