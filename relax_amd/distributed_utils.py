"""Drop-in counterpart of ``distributed_masked_whiten`` (relax/utils/distributed_utils.py:98-158) on one GPU."""

from __future__ import annotations

import torch

from . import ops


def distributed_masked_whiten(values, mask, process_group=None, shift_mean: bool = True, epsilon: float = 1e-8):
    """Masked mean / Bessel-corrected variance whitening.  ``process_group`` must be None or a single rank: the
    statistics are those of this GPU's data.  Raises ``ValueError`` when the mask sums to zero (one host read of
    the mask sum, as the reference's ``.item()``)."""
    if process_group is not None and hasattr(process_group, "size") and process_group.size() > 1:
        raise NotImplementedError("multi-rank whitening is outside the one-GPU path")
    out, stats = ops.masked_whiten(values, mask, shift_mean, epsilon)
    if stats[2].item() == 0:
        raise ValueError("The global mask sum across all participating GPUs is zero.")
    return out.reshape(values.shape)
