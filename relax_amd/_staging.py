"""Asynchronous upload of small host integer arrays (sample offsets, row starts).

A plain ``torch.tensor(list).to(device)`` is a pageable copy: it blocks the host until every kernel queued before it
has finished, which stalls the launch pipeline once per micro-batch.  This module keeps a small per-thread ring of
pinned buffers; each upload is a ``non_blocking`` copy guarded by an event, so a slot is only rewritten after the copy
that last used it has completed.
"""

from __future__ import annotations

import threading

import torch

_SLOTS = 8
_CAPACITY = 1 << 14  # int64 elements per slot

_local = threading.local()


class _Slot:
    __slots__ = ("buf", "event")

    def __init__(self):
        self.buf = torch.empty(_CAPACITY, dtype=torch.int64, pin_memory=True)
        self.event = None


def upload_int64(values, device) -> torch.Tensor:
    """Device int64 tensor holding ``values`` (a list of Python ints or a CPU tensor), without a host-side sync."""
    host = values if isinstance(values, torch.Tensor) else torch.tensor(values, dtype=torch.int64)
    host = host.to(torch.int64).reshape(-1)
    n = host.numel()
    if n > _CAPACITY or n == 0:
        return host.to(device)
    ring = getattr(_local, "ring", None)
    if ring is None:
        ring = _local.ring = {"slots": [_Slot() for _ in range(_SLOTS)], "next": 0}
    slot = ring["slots"][ring["next"]]
    ring["next"] = (ring["next"] + 1) % _SLOTS
    if slot.event is not None:
        slot.event.synchronize()
    slot.buf[:n].copy_(host)
    out = slot.buf[:n].to(device, non_blocking=True)
    slot.event = torch.cuda.Event()
    slot.event.record(torch.cuda.current_stream(device))
    return out
