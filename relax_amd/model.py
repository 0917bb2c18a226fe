"""Caller side of the fused LM head: make the model return hidden states and hand the loss the LM-head operand.

Counterpart of ``_find_lm_output_layer`` / ``_bypass_output_layer`` (relax/backends/megatron/model.py:63-181).  The
reference swaps ``output_layer.forward`` for a passthrough during the model forward and yields a closure that runs the
real projection per 1024-row sub-chunk.  Here the yielded object is still such a callable (so code written against the
reference keeps working), but it also exposes ``.weight`` -- the explicit weight the model passed to the deferred call
(tied embeddings) or the layer's own -- which is what ``get_log_probs_and_entropy(..., lm_head_forward=...)`` and
``sft_loss_function_chunked`` feed to the matrix-core kernel instead of calling it.

One GPU: tensor-parallel size 1, so there is no sequence-parallel gather; a layer with ``sequence_parallel`` set is
refused rather than silently mishandled.
"""

from __future__ import annotations

from contextlib import contextmanager
from typing import Iterator

import torch


def find_lm_output_layer(model: torch.nn.Module) -> torch.nn.Module | None:
    """The LM head behind DDP-style ``.module`` wrappers and multimodal ``.language_model`` bridges; ``None`` when the
    model has none or only the ``nn.Identity`` placeholder of a non-last pipeline stage (model.py:63-92; the walk is
    bounded like the reference's)."""
    module = model
    for _ in range(5):
        head = getattr(module, "output_layer", None)
        if head is not None and not isinstance(head, torch.nn.Identity):
            return head
        module = getattr(module, "module", None) or getattr(module, "language_model", None)
        if module is None:
            return None
    return None


class DeferredLMHead:
    """What ``bypass_output_layer`` yields: callable like the reference's closure, and a carrier of the operand."""

    def __init__(self, output_layer: torch.nn.Module, original_forward):
        self.output_layer = output_layer
        self._forward = original_forward
        self._explicit_weight = None
        self.deferred = False

    @property
    def weight(self) -> torch.Tensor:
        w = self._explicit_weight if self._explicit_weight is not None else getattr(self.output_layer, "weight", None)
        if w is None:
            raise RuntimeError("Unable to resolve lm_head weight for chunked SFT loss")
        return w

    @property
    def bias(self):
        return getattr(self.output_layer, "bias", None)

    def __call__(self, input_, weight=None, runtime_gather_output=None):
        """The real projection (model.py:145-161): input cast to the weight dtype; returns what the layer returns."""
        call_weight = weight if weight is not None else self._explicit_weight
        w = call_weight if call_weight is not None else getattr(self.output_layer, "weight", None)
        if w is None:
            raise RuntimeError("Unable to resolve lm_head weight for chunked SFT loss")
        if input_.dtype != w.dtype:
            input_ = input_.to(w.dtype)
        return self._forward(input_, weight=call_weight, runtime_gather_output=runtime_gather_output)


@contextmanager
def bypass_output_layer(model: torch.nn.Module, *, mtp_output_layer_calls: int = 0) -> Iterator[DeferredLMHead | None]:
    """Inside the block the model's main LM-head call returns ``(hidden_states, None)`` unchanged.

    The first ``mtp_output_layer_calls`` calls (multi-token-prediction depths use the same layer before the main head)
    go to the real layer; the next one is deferred; a further one is an error, and so is leaving the block without the
    main call having happened.  The original forward is restored on exit, exception or not.  Yields ``None`` (and does
    nothing) when the model has no LM head."""
    assert mtp_output_layer_calls >= 0, f"{mtp_output_layer_calls=}"
    head = find_lm_output_layer(model)
    if head is None:
        yield None
        return
    if bool(getattr(head, "sequence_parallel", False)):
        raise NotImplementedError("bypass_output_layer: a sequence-parallel LM head needs a tensor-parallel gather; "
                                  "this build runs at tensor-parallel size 1")
    original_forward = head.forward
    deferred = DeferredLMHead(head, original_forward)
    remaining_mtp = mtp_output_layer_calls

    def passthrough(input_, weight=None, runtime_gather_output=None, **kwargs):
        nonlocal remaining_mtp
        if remaining_mtp > 0:
            remaining_mtp -= 1
            return original_forward(input_, weight=weight, runtime_gather_output=runtime_gather_output, **kwargs)
        if deferred.deferred:
            raise RuntimeError("output_layer was called more than once after all MTP head calls")
        deferred.deferred = True
        deferred._explicit_weight = weight
        return input_, None

    head.forward = passthrough
    try:
        yield deferred
        if not deferred.deferred:
            observed = mtp_output_layer_calls - remaining_mtp
            raise RuntimeError("The main output_layer was not reached after the configured MTP head calls: "
                               f"{mtp_output_layer_calls=}, observed_mtp_calls={observed}")
    finally:
        try:
            del head.forward  # drop the instance attribute: the class's forward shows through again
        except AttributeError:
            head.forward = original_forward
