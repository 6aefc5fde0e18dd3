"""CPU: a converted linear traces under ``torch.compile(fullgraph=True)`` as opaque operators.

The reference compiles each transformer block as a whole graph
(torchtitan/models/llama3/parallelize.py:271-284); here the tracing half of that is checked
without a GPU: Dynamo must follow ``F.linear`` on the wrapped weight into the registered operator
without a graph break, and the fake kernels must give the shapes the real ones produce.  The
backend used records the graph and refuses to run it (the operators have GPU kernels only)."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from torchtitan_amd import compiled  # registers torchtitan_amd::mx_linear_fwd / _bwd
from torchtitan_amd import ops
from torchtitan_amd.modules import FeedForward, Linear
from torchtitan_amd.mx_tensor import MXFP8Config, MXFP8TrainingWeight, wrap_parameter


class _Recorded(Exception):
    pass


def _trace(module, *inputs):
    graphs = []

    def backend(gm, example_inputs):
        graphs.append(gm)

        def refuse(*args):
            raise _Recorded()
        return refuse

    fn = torch.compile(module, backend=backend, fullgraph=True)
    with pytest.raises(_Recorded):
        fn(*inputs)
    assert len(graphs) == 1, "one graph, no break"
    return graphs[0]


_FWD = (torch.ops.torchtitan_amd.mx_linear_fwd, torch.ops.torchtitan_amd.mx_linear_fwd.default)


def _targets(gm):
    return [n.target for n in gm.graph.nodes if n.op == "call_function"]


def _count_fwd(gm):
    return sum(t in _FWD for t in _targets(gm))


def test_converted_linear_traces_as_one_operator():
    lin = Linear.Config(bias=True).build(in_features=64, out_features=96)
    lin.weight = wrap_parameter(lin.weight, MXFP8Config("rceil"))
    gm = _trace(lin, torch.randn(2, 32, 64))
    assert _count_fwd(gm) == 1
    assert F.linear not in _targets(gm) and torch._C._nn.linear not in _targets(gm)
    # the operator's first output is what the module returns (plus the bias add)
    node = next(n for n in gm.graph.nodes if n.target in _FWD)
    assert node.args[2] == ops.SCALE_MODES["rceil"]
    y, xc, xs, wc, ws = node.meta["example_value"]
    assert y.shape == (2, 32, 96) and y.dtype == torch.bfloat16
    assert xc.shape == (64, 64) and wc.shape == (64, 96) and xc.dtype == torch.uint8
    assert xs.numel() == ops.mfma_scale_bytes(64, 2) and ws.numel() == ops.mfma_scale_bytes(64, 3)


def test_feed_forward_block_traces_as_three_operators():
    """Under a tracer the block takes the three-linears route (the fused block functions are
    eager-only), silu and the product stay ordinary graph nodes."""
    ff = FeedForward.Config(hidden_dim=128).build(dim=64)
    for lin in (ff.w1, ff.w2, ff.w3):
        lin.weight = wrap_parameter(lin.weight, MXFP8Config("floor"))
    gm = _trace(ff, torch.randn(32, 64))
    t = _targets(gm)
    assert _count_fwd(gm) == 3
    assert any("silu" in str(x) for x in t)


def test_fake_kernels_reject_unaligned_shapes_and_give_backward_shapes():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        x, w = torch.empty(64, 64), torch.empty(96, 64)
        y, xc, xs, wc, ws = torch.ops.torchtitan_amd.mx_linear_fwd(x, w, 1)
        dx, dw = torch.ops.torchtitan_amd.mx_linear_bwd(torch.empty(64, 96), xc, xs, wc, ws, 1, True, True)
        assert dx.shape == (64, 64) and dw.shape == (96, 64) and dx.dtype == torch.bfloat16
        dx, dw = torch.ops.torchtitan_amd.mx_linear_bwd(torch.empty(64, 96), xc, xs, wc, ws, 1, False, True)
        assert dx.numel() == 0 and dw.shape == (96, 64)
        with pytest.raises(Exception):
            torch.ops.torchtitan_amd.mx_linear_fwd(torch.empty(40, 64), w, 1)


def test_operators_have_no_cpu_kernel():
    """No fallback: off the GPU the operators fail instead of computing something else."""
    with pytest.raises(Exception):
        torch.ops.torchtitan_amd.mx_linear_fwd(torch.randn(32, 64), torch.randn(32, 64), 1)
