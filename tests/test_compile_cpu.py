"""CPU: converted linears and grouped experts trace under ``torch.compile(fullgraph=True)`` as
opaque operators.

The reference compiles each transformer block as a whole graph
(torchtitan/models/llama3/parallelize.py:271-284); here the tracing half of that is checked
without a GPU: Dynamo must follow ``F.linear`` on the wrapped weight into the registered operator
without a graph break, and the fake kernels must give the shapes the real ones produce.  The
backend used records the graph and refuses to run it (the operators have GPU kernels only)."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from torchtitan_amd import compiled  # registers the torchtitan_amd:: traced operators
from torchtitan_amd import ops
from torchtitan_amd.modules import FeedForward, GroupedExperts, Linear
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
    gm = _trace(lin, torch.randn(2, 32, 64, requires_grad=True))
    assert _count_fwd(gm) == 1
    assert F.linear not in _targets(gm) and torch._C._nn.linear not in _targets(gm)
    # the operator's first output is what the module returns (plus the bias add)
    node = next(n for n in gm.graph.nodes if n.target in _FWD)
    assert node.args[2] == ops.SCALE_MODES["rceil"] and node.args[3:5] == (True, True)
    y, xc, xs, wc, ws = node.meta["example_value"]
    assert y.shape == (2, 32, 96) and y.dtype == torch.bfloat16
    assert xc.shape == (64, 64) and wc.shape == (64, 96) and xc.dtype == torch.uint8
    assert xs.numel() == ops.mfma_scale_bytes(64, 2) and ws.numel() == ops.mfma_scale_bytes(64, 3)


def test_traced_linear_leaves_out_the_casts_no_gradient_needs():
    """An input that needs no gradient: no column-wise form of W is made or kept; under no_grad
    none of x either."""
    lin = Linear.Config(bias=False).build(in_features=64, out_features=96)
    lin.weight = wrap_parameter(lin.weight, MXFP8Config("rceil"))
    gm = _trace(lin, torch.randn(32, 64))
    node = next(n for n in gm.graph.nodes if n.target in _FWD)
    assert node.args[3:5] == (False, True)
    _, xc, xs, wc, ws = node.meta["example_value"]
    assert xc.shape == (64, 32) and wc.numel() == 0 and ws.numel() == 0

    class NoGrad(nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = lin

        def forward(self, x):
            with torch.no_grad():
                return self.lin(x)

    gm = _trace(NoGrad(), torch.randn(32, 64))
    node = next(n for n in gm.graph.nodes if n.target in _FWD)
    assert node.args[3:5] == (False, False)
    assert all(t.numel() == 0 for t in node.meta["example_value"][1:])


def test_weights_converted_before_the_dtype_change_still_trace():
    """The reference converts first and moves / casts the model afterwards
    (torchtitan/trainer.py:272-276 then :399-418): ``module.to(dtype)`` swaps the data of the
    converted parameter in place, and nothing of the parameter may keep the old dtype (a tracer
    compares a tensor and its base with their fake twins)."""
    lin = Linear.Config().build(in_features=64, out_features=96)
    lin.weight = wrap_parameter(lin.weight, MXFP8Config("rceil"))
    assert isinstance(lin.weight, nn.Parameter) and lin.weight._base is None
    lin.to(torch.bfloat16)
    assert lin.weight.dtype == torch.bfloat16 and isinstance(lin.weight, MXFP8TrainingWeight)
    gm = _trace(lin, torch.randn(32, 64, dtype=torch.bfloat16))
    assert _count_fwd(gm) == 1


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


_GFWD = (torch.ops.torchtitan_amd.mx_grouped_mm_fwd, torch.ops.torchtitan_amd.mx_grouped_mm_fwd.default)
_PLAN = (torch.ops.torchtitan_amd.group_offsets_pad, torch.ops.torchtitan_amd.group_offsets_pad.default)


def _experts(pad, dim=128, hidden=256, n=4):
    ex = GroupedExperts(dim=dim, hidden_dim=hidden, num_experts=n, use_grouped_mm=True)
    for name in ("w1", "w2", "w3"):
        setattr(ex, name, wrap_parameter(getattr(ex, name), MXFP8Config("rceil", pad_token_groups_for_grouped_mm=pad)))
    return ex


@pytest.mark.parametrize("pad", [True, False])
def test_grouped_experts_trace_as_three_grouped_operators(pad):
    """The tracer does not offer ``torch._grouped_mm`` to a tensor subclass (underscore names are
    not among the overridable functions), so the expert block calls the package's
    ``grouped_mm``: three MXFP8 operators in one graph and no bf16 ``_grouped_mm`` left.
    Experts that pad their groups themselves need no padding wrapper around them; the others
    keep the wrapper, whose index fill is a graph node too."""
    gm = _trace(_experts(pad), torch.randn(96, 128), torch.tensor([10, 40, 30, 16]))
    t = _targets(gm)
    assert sum(x in _GFWD for x in t) == 3
    assert torch._grouped_mm not in t
    assert sum(x in _PLAN for x in t) == (0 if pad else 1)
    node = next(n for n in gm.graph.nodes if n.target in _GFWD)
    assert node.args[3] == ops.SCALE_MODES["rceil"] and node.args[4] is pad


@pytest.mark.parametrize("T,K,N,G,pad", [(96, 128, 256, 4, True), (96, 128, 256, 4, False),
                                         (100, 96, 160, 3, True), (96, 96, 160, 3, False)])
def test_grouped_fake_kernels_give_the_static_shapes(T, K, N, G, pad):
    from torch._subclasses.fake_tensor import FakeTensorMode

    fast = K % 128 == 0 and N % 128 == 0
    padded = pad or fast
    step = 128 if fast else 32
    Tp = -(-(T + 32 * G) // step) * step if padded else T
    with FakeTensorMode():
        x, w, offs = torch.empty(T, K), torch.empty(G, N, K), torch.empty(G, dtype=torch.int32)
        y, offs_p, perm, back, xc, xs, wc, ws = torch.ops.torchtitan_amd.mx_grouped_mm_fwd(x, w, offs, 1, pad)
        assert y.shape == (T, N) and y.dtype == torch.bfloat16 and offs_p.shape == (G,)
        assert perm.shape == ((Tp,) if padded else (0,))
        # the way back: the unpadded group ends where the GEMM writes unpadded rows, else a gather
        assert (back.shape, back.dtype) == (((G,), torch.int32) if fast else ((T,) if padded else (0,), torch.int64))
        assert xc.shape == (K, Tp) and wc.shape == (G, K, N)
        assert xs.shape == ((ops.mfma_scale_bytes(K, Tp // 32),) if fast else (K, Tp // 32))
        assert ws.numel() == G * ops.mfma_scale_bytes(K, N // 32)
        dx, dw = torch.ops.torchtitan_amd.mx_grouped_mm_bwd(torch.empty(T, N), offs_p, perm, back, xc, xs, wc, ws,
                                                            1, True, True)
        assert dx.shape == (T, K) and dw.shape == (G, N, K)
        dx, dw = torch.ops.torchtitan_amd.mx_grouped_mm_bwd(torch.empty(T, N), offs_p, perm, back, xc, xs, wc, ws,
                                                            1, True, False)
        assert dx.shape == (T, K) and dw.numel() == 0
        with pytest.raises(Exception):
            torch.ops.torchtitan_amd.mx_grouped_mm_fwd(torch.empty(T, 40), torch.empty(G, N, 40), offs, 1, pad)


def test_fused_block_fake_kernels_give_the_shapes_the_backward_takes():
    """The fused block operators (feed-forward, expert block, routed experts): fake forward
    outputs feed the fake backward, with and without the parts no gradient asks for."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    A = torch.ops.torchtitan_amd
    with FakeTensorMode():
        x, w1, w2 = torch.empty(2, 64, 128, dtype=torch.bfloat16), torch.empty(256, 128), torch.empty(128, 256)
        out = A.mx_ffn_fwd(x, w1, w2, w1, None, 0.0, 1, False, True, True)
        assert len(out) == 15 and out[0].shape == (2, 64, 128) and out[1].shape == (2, 128, 256)
        assert out[4].shape == (128, 128) and out[8].shape == (128, 256)
        dx, dw13, dw2, dnw = A.mx_ffn_bwd(torch.empty(2, 64, 128), list(out[1:]), None, None, 1, True, True, True, True, False)
        assert dx.shape == (128, 128) and dw13.shape == (2, 256, 128) and dw2.shape == (128, 256) and dnw.numel() == 0
        out = A.mx_ffn_fwd(x, w1, w2, w1, None, 0.0, 1, False, False, False)
        assert all(t.numel() == 0 for t in out[1:])
        nw = torch.empty(128, dtype=torch.bfloat16)
        out = A.mx_ffn_fwd(x, w1, w2, w1, nw, 1e-5, 1, False, True, True)
        assert out[13].shape == (128,) and out[12].numel() == 0 and out[14].numel() == 0
        dx, _, _, dnw = A.mx_ffn_bwd(torch.empty(2, 64, 128), list(out[1:]), x, nw, 1, True, True, True, True, True)
        assert dx.shape == (128, 128) and dnw.shape == (128,)
        with pytest.raises(Exception):
            A.mx_ffn_fwd(torch.empty(40, 128), w1, w2, w1, None, 0.0, 1, False, True, True)

        T, D, H, G, k = 96, 128, 256, 4, 2
        xg, e1, e2 = torch.empty(T, D, dtype=torch.bfloat16), torch.empty(G, H, D), torch.empty(G, D, H)
        offs = torch.empty(G, dtype=torch.int32)
        Tp = -(-(T + 32 * G) // 128) * 128
        out = A.mx_grouped_ffn_fwd(xg, e1, e2, e1, offs, 1, True, False, True, True)
        assert out[0].shape == (T, D) and out[2].shape == (Tp,) and out[4].shape == (2, Tp, H)
        assert out[3].shape == (G,) and out[3].dtype == torch.int32  # the unpadded group ends: the GEMMs write unpadded rows
        dx, dw13, dw2 = A.mx_grouped_ffn_bwd(torch.empty(T, D), list(out[1:]), 1, ops.MX_SCALES_MFMA, True, True, True, False)
        assert dx.shape == (T, D) and dw13.shape == (1, G, H, D) and dw2.shape == (G, D, H)

        scores, order, counts = torch.empty(T, k), torch.empty(T * k, dtype=torch.int64), torch.empty(G, dtype=torch.int64)
        Tp = -(-(T * k + 32 * G) // 128) * 128
        for before in (True, False):
            out = A.mx_routed_experts_fwd(xg, scores, e1, e2, e1, order, counts, before, 1, False, True, True, True)
            assert len(out) == 18 and out[0].shape == (T, D) and out[4].shape == (T, k) and out[6].shape == (2, Tp, H)
            assert out[17].shape == ((0,) if before else (Tp, D))
            dx, ds, dw13, dw2 = A.mx_routed_experts_bwd(torch.empty(T, D), list(out[1:]), xg if before else None, 1,
                                                        ops.MX_SCALES_MFMA, before, True, True, True, True, True)
            assert dx.shape == (T, D) and ds.shape == (T, k) and ds.dtype == torch.float32 and dw13.shape == (2, G, H, D)


def test_operators_have_no_cpu_kernel():
    """No fallback: off the GPU the operators fail instead of computing something else."""
    with pytest.raises(Exception):
        torch.ops.torchtitan_amd.mx_linear_fwd(torch.randn(32, 64), torch.randn(32, 64), 1)
    with pytest.raises(Exception):
        torch.ops.torchtitan_amd.mx_grouped_mm_fwd(torch.randn(32, 64), torch.randn(2, 32, 64),
                                                   torch.tensor([16, 32], dtype=torch.int32), 1, True)
    with pytest.raises(Exception):
        torch.ops.torchtitan_amd.group_offsets_pad(torch.tensor([3, 5]), 2, 1, 64, 32)
