"""Drop-in counterparts of the masked reducers of ``relax/backends/megatron/cp_utils.py`` at context-parallel
size 1 (reference lines :125-162 reducers, :209-285 token counts), on the gfx950 segment-sum kernel."""

from __future__ import annotations

import torch

from . import ops
from ._staging import upload_int64


def _cu(response_lengths, device) -> torch.Tensor:
    cu = [0]
    for r in response_lengths:
        cu.append(cu[-1] + int(r))
    return upload_int64(cu, device)


def _mask_sums(loss_masks, cu_resp=None) -> torch.Tensor:
    """Exact per-sample mask sums (fp64 accumulation in the kernel), returned in the masks' own dtype."""
    dev = loss_masks[0].device
    if cu_resp is None:
        cu_resp = _cu([m.numel() for m in loss_masks], dev)
    sums = ops.segment_sum(torch.cat([m.reshape(-1) for m in loss_masks]), cu_resp)
    dt = loss_masks[0].dtype
    return sums.round().to(dt) if not dt.is_floating_point else sums.to(dt)


def sample_denominators(loss_masks, layout=None, sample_denoms=None) -> torch.Tensor:
    """fp32 [B] divisors ``clamp_min(denom_i, 1)`` of the sample-mean reducer (cp_utils.py:138-149)."""
    dev = loss_masks[0].device
    if sample_denoms is None:
        den = _mask_sums(loss_masks, None if layout is None else layout.cu_resp)
    else:
        den = torch.as_tensor(sample_denoms, device=dev)
    return torch.clamp_min(den, 1).to(torch.float32)


class _MaskedSampleReduce(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, mask, cu_resp, inv_den):
        sums = ops.segment_sum(mask, cu_resp, values=x)
        ctx.save_for_backward(mask, cu_resp, inv_den)
        ctx.n, ctx.dtype = x.numel(), x.dtype
        return (sums.to(torch.float32) * inv_den).sum().to(x.dtype if x.dtype.is_floating_point else torch.float32)

    @staticmethod
    def backward(ctx, g):
        mask, cu_resp, inv_den = ctx.saved_tensors
        per_tok = ops.broadcast_per_sample(inv_den, cu_resp, ctx.n)
        return (per_tok * mask * g.to(torch.float32)).to(ctx.dtype), None, None, None


def get_sum_of_sample_mean(
    total_lengths,
    response_lengths,
    loss_masks,
    calculate_per_token_loss: bool = False,
    qkv_format: str = "thd",
    max_seq_lens=None,
    padded_total_lengths=None,
    dynamic_cp_size=None,
    dynamic_cp_rank=None,
    sample_denoms=None,
):
    """Returns the reducer ``x [N] -> scalar``: sum over samples of the masked mean (or the masked token sum)."""
    if dynamic_cp_size not in (None, 1):
        raise NotImplementedError("context parallelism is outside the one-GPU path")
    dev = loss_masks[0].device
    cu = _cu(response_lengths, dev)
    mask = torch.cat([m.reshape(-1) for m in loss_masks]).to(torch.float32)
    if calculate_per_token_loss:
        inv = torch.ones(len(response_lengths), dtype=torch.float32, device=dev)
    else:
        inv = 1.0 / sample_denominators(loss_masks, None, sample_denoms)

    def reducer(x: torch.Tensor) -> torch.Tensor:
        return _MaskedSampleReduce.apply(x, mask, cu, inv)

    reducer.relax_amd_linear = True  # a fixed weighted sum of its argument: callers may read the weights off it
    return reducer


class PerSampleDivisorReducer:
    """Reducer ``x [N] -> sum_i (x_i * m_i).sum() / divisor_i`` that also carries its divisors.

    A function named by ``--custom-pg-loss-reducer-function-path`` (loss.py:1062-1072) may return one of these instead
    of an opaque callable: ``policy_loss_function`` then reads ``sample_divisors`` and evaluates the pg_loss reduction
    inside its fused launch; any other code can still call the object like the closure the reference expects."""

    relax_amd_linear = True  # a fixed weighted sum of its argument

    def __init__(self, response_lengths, loss_masks, sample_divisors):
        self.response_lengths = [int(r) for r in response_lengths]
        self.loss_masks = loss_masks
        self.sample_divisors = torch.as_tensor(sample_divisors, dtype=torch.float32).reshape(-1)
        if self.sample_divisors.numel() != len(self.response_lengths):
            raise ValueError(f"{self.sample_divisors.numel()} divisors for {len(self.response_lengths)} samples")
        self._state = None

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        if self._state is None or self._state[0].device != x.device:
            dev = x.device
            mask = torch.cat([m.reshape(-1) for m in self.loss_masks]).to(device=dev, dtype=torch.float32)
            self._state = (mask, _cu(self.response_lengths, dev), 1.0 / self.sample_divisors.to(dev))
        return _MaskedSampleReduce.apply(x, *self._state)


def get_seq_mean_token_sum_reducer(total_lengths, response_lengths, loss_masks, calculate_per_token_loss=False):
    """``--custom-pg-loss-reducer-function-path relax_amd.cp_utils.get_seq_mean_token_sum_reducer``: every sequence's
    masked token sum, averaged over the B sequences of the micro-batch (sequence-mean of token-sums; a fully masked
    sequence still counts in B).  Signature of the reference's plug-in point, loss.py:1066-1068."""
    b = len(response_lengths)
    return PerSampleDivisorReducer(response_lengths, loss_masks, torch.full((b,), float(max(b, 1))))


def get_cp_local_mask_sums(total_lengths, response_lengths, loss_masks, qkv_format="thd", max_seq_lens=None,
                           padded_total_lengths=None, dynamic_cp_size=None, dynamic_cp_rank=None) -> torch.Tensor:
    return _mask_sums(loss_masks)


def get_cp_local_num_tokens(total_lengths, response_lengths, loss_masks, qkv_format="thd", max_seq_lens=None,
                            padded_total_lengths=None, dynamic_cp_size=None, dynamic_cp_rank=None) -> torch.Tensor:
    """``sum_i clamp_min(sum(mask_i), 1)`` -- a fully masked sample counts as one token (cp_utils.py:283-285)."""
    return torch.clamp_min(_mask_sums(loss_masks), 1).sum()
