"""Deferred-LM-head plumbing on the caller side (CPU): the behaviours the reference's own tests require of
``_bypass_output_layer`` / ``_find_lm_output_layer`` (tests/backends/megatron/test_sft_chunked_ce.py:141-399), against
stand-in layers written here."""

import pytest
import torch
import torch.nn.functional as F

from relax_amd.loss import lm_head_weight_of
from relax_amd.model import bypass_output_layer, find_lm_output_layer


class Head(torch.nn.Module):
    """Column-parallel-linear look-alike: forward(input, weight=None, runtime_gather_output=None) -> (out, bias)."""

    def __init__(self, h=4, v=8):
        super().__init__()
        self.weight = torch.nn.Parameter(torch.randn(v, h) * 0.02)
        self.sequence_parallel = False

    def forward(self, input_, weight=None, runtime_gather_output=None):
        return F.linear(input_, self.weight if weight is None else weight), None


class Model(torch.nn.Module):
    def __init__(self, head=None):
        super().__init__()
        self.output_layer = head if head is not None else Head()


class Wrapper(torch.nn.Module):
    def __init__(self, inner):
        super().__init__()
        self.module = inner


class Bridge(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.language_model = Model()


def test_find_output_layer_plain_wrapped_bridged_absent_and_placeholder():
    m = Model()
    assert find_lm_output_layer(m) is m.output_layer
    b = Bridge()
    assert find_lm_output_layer(Wrapper(b)) is b.language_model.output_layer
    assert find_lm_output_layer(Wrapper(Wrapper(m))) is m.output_layer
    assert find_lm_output_layer(torch.nn.Linear(2, 2)) is None
    assert find_lm_output_layer(Model(torch.nn.Identity())) is None  # non-last pipeline stage


def test_passthrough_inside_real_projection_from_the_handle_and_restored_after():
    m = Model()
    x = torch.randn(3, 4)
    want = x @ m.output_layer.weight.t()
    with bypass_output_layer(m) as head:
        y, bias = m.output_layer(x)
        assert torch.equal(y, x) and bias is None
        z, _ = head(x)
        torch.testing.assert_close(z, want)
        assert head.weight is m.output_layer.weight and lm_head_weight_of(head) is m.output_layer.weight
    torch.testing.assert_close(m.output_layer(x)[0], want)
    assert "forward" not in vars(m.output_layer)


def test_mtp_calls_use_the_real_head_and_only_the_main_call_is_deferred():
    m = Model()
    x = torch.randn(3, 4)
    want = x @ m.output_layer.weight.t()
    with bypass_output_layer(m, mtp_output_layer_calls=2) as head:
        torch.testing.assert_close(m.output_layer(x)[0], want)
        torch.testing.assert_close(m.output_layer(x)[0], want)
        hidden, bias = m.output_layer(x)
        assert torch.equal(hidden, x) and bias is None
        torch.testing.assert_close(head(hidden)[0], want)
        with pytest.raises(RuntimeError, match="more than once"):
            m.output_layer(x)
    # functional_call on the layer with detached parameters counts as one of the MTP calls
    detached = {k: p.detach() for k, p in m.output_layer.named_parameters()}
    with bypass_output_layer(m, mtp_output_layer_calls=1) as head:
        mtp, _ = torch.func.functional_call(m.output_layer, detached, (x,), {"runtime_gather_output": None})
        hidden, _ = m.output_layer(x)
        main, _ = head(hidden)
    torch.testing.assert_close(mtp, want)
    torch.testing.assert_close(main, want)


def test_missing_main_call_is_an_error_and_forward_is_restored_even_after_exceptions():
    m = Model()
    x = torch.randn(3, 4)
    with pytest.raises(RuntimeError, match="main output_layer was not reached"):
        with bypass_output_layer(m, mtp_output_layer_calls=1):
            m.output_layer(x)  # consumed as the MTP call; the main call never happens
    torch.testing.assert_close(m.output_layer(x)[0], x @ m.output_layer.weight.t())
    with pytest.raises(RuntimeError, match="boom"):
        with bypass_output_layer(m):
            raise RuntimeError("boom")
    torch.testing.assert_close(m.output_layer(x)[0], x @ m.output_layer.weight.t())


def test_tied_embeddings_weight_is_taken_from_the_deferred_call():
    class Tied(torch.nn.Module):
        weight = None
        sequence_parallel = False

        def forward(self, input_, weight=None, runtime_gather_output=None):
            assert weight is not None
            return F.linear(input_, weight), None

    m = Model(Tied())
    shared = torch.nn.Parameter(torch.randn(8, 4))
    x = torch.randn(3, 4)
    with bypass_output_layer(m) as head:
        with pytest.raises(RuntimeError, match="Unable to resolve lm_head weight"):
            head.weight  # nothing known before the model's own call
        hidden, _ = m.output_layer(x, weight=shared)
        assert head.weight is shared and lm_head_weight_of(head) is shared
        torch.testing.assert_close(head(hidden)[0], x @ shared.t())


def test_no_output_layer_yields_none_dtype_alignment_and_sequence_parallel_refused():
    with bypass_output_layer(torch.nn.Linear(2, 2)) as head:
        assert head is None
    m = Model()
    m.output_layer.weight.data = m.output_layer.weight.data.to(torch.bfloat16)
    with bypass_output_layer(m) as head:
        hidden, _ = m.output_layer(torch.randn(3, 4))  # fp32 hidden states from an upcasting bridge
        y, _ = head(hidden)
    assert y.dtype == torch.bfloat16 and y.shape == (3, 8)
    sp = Model()
    sp.output_layer.sequence_parallel = True
    with pytest.raises(NotImplementedError, match="tensor-parallel"):
        with bypass_output_layer(sp):
            pass
    with pytest.raises(AssertionError):
        with bypass_output_layer(Model(), mtp_output_layer_calls=-1):
            pass
