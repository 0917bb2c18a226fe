"""Drop-in counterpart of ``distributed_masked_whiten`` (relax/utils/distributed_utils.py:98-158) on one GPU."""

from __future__ import annotations

import torch

from . import _lib, ops


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


def distributed_masked_normalize(values, mask, process_group=None, variance_floor: float = 1e-8):
    """REINFORCE++ normaliser on one rank (relax/utils/distributed_utils.py:161-213): population mean / variance
    (ddof = 0) over ``mask != 0``, output explicitly zero outside the mask.  Returns ``(normalized, mean, variance,
    count)`` with 0-d moment tensors; no host synchronisation (an all-zero mask yields count 0 and zeros)."""
    if process_group is not None and hasattr(process_group, "size") and process_group.size() > 1:
        raise NotImplementedError("multi-rank normalisation is outside the one-GPU path")
    if values.shape != mask.shape:
        raise ValueError(f"values and mask must have the same shape, got {values.shape} and {mask.shape}.")
    if variance_floor <= 0:
        raise ValueError(f"variance_floor must be positive, got {variance_floor}.")
    dev = ops._need_gpu(values)
    dtype, code = (torch.float64, _lib.F64) if values.dtype == torch.float64 else (torch.float32, _lib.F32)
    v = values.reshape(-1).to(dtype).contiguous()
    m = mask.reshape(-1).to(device=dev, dtype=dtype).contiguous()
    out = torch.empty_like(v)
    stats = torch.empty(3, dtype=dtype, device=dev)
    _lib.check(_lib.lib.relax_amd_masked_normalize(ops._p(v), ops._p(m), code, v.numel(), float(variance_floor),
                                                   ops._p(out), ops._p(stats), ops._stream()))
    return out.reshape(values.shape), stats[0], stats[1], stats[2]
