"""GPU: the converted blocks inside a captured HIP graph.

Nothing on the MXFP8 path synchronises with the host or clears memory with a memset (group
sizes stay on the device, padded lengths are static bounds, flags are cleared by fill kernels),
so a forward + backward through converted modules can be captured once and replayed.  Each test
replays the graph several times on new inputs, with eager work and synchronisations between the
replays, and checks every replay bit for bit against the eager run of the same step.  No test
clears the activation-cast reuse by hand: an entry made by the eager warm-up must not be taken
under capture (the cast would be missing from the graph and every replay would reuse old codes)."""
import pytest
import torch
import torch.nn as nn

from torchtitan_amd.modules import FeedForward, Linear, MoE
from torchtitan_amd.protocols import ModelConvertersContainer
from torchtitan_amd.quantization.mx import MXFP8Converter

pytestmark = pytest.mark.gpu


def _convert(model, fqns):
    ModelConvertersContainer.Config(
        converters=[MXFP8Converter.Config(fqns=fqns, recipe_name="mxfp8_rceil")]
    ).build(parallel_dims=None, model_compile_enabled=False).convert(model)


def _step(module, x, dy):
    for p in module.parameters():
        p.grad = None
    x.grad = None
    module(x).backward(dy)


def _results(module, x):
    return [x.grad.clone()] + [p.grad.clone() for p in module.parameters() if p.grad is not None]


def _check_graph_replays(module, shape, device):
    inputs = [(torch.randn(shape, device=device, dtype=torch.bfloat16),
               torch.randn(shape, device=device, dtype=torch.bfloat16)) for _ in range(3)]
    x = torch.zeros(shape, device=device, dtype=torch.bfloat16, requires_grad=True)
    dy = torch.zeros(shape, device=device, dtype=torch.bfloat16)
    eager = []
    for xi, dyi in inputs:
        with torch.no_grad():
            x.copy_(xi)
            dy.copy_(dyi)
        _step(module, x, dy)
        eager.append(_results(module, x))
    # warm-up on a side stream (first-call set-up of the library happens here), then capture
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _step(module, x, dy)
    torch.cuda.current_stream().wait_stream(side)
    for p in module.parameters():
        p.grad = None
    x.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        module(x).backward(dy)
    for rep in range(2):
        for (xi, dyi), want in zip(inputs, eager):
            with torch.no_grad():
                x.copy_(xi)
                dy.copy_(dyi)
            graph.replay()
            torch.cuda.synchronize()
            got = _results(module, x)
            scratch = torch.randn(1 << 20, device=device).sum().item()  # eager work between replays
            assert scratch == scratch
            assert len(got) == len(want)
            for g, w in zip(got, want):
                assert torch.equal(g, w), (rep, g.shape)


def test_swiglu_block_in_a_captured_graph(device):
    torch.manual_seed(31)
    ff = FeedForward.Config(hidden_dim=512).build(dim=256).to(device).to(torch.bfloat16)
    ff.init_weights(init_std=0.05)
    holder = nn.Module()
    holder.feed_forward = ff
    _convert(holder, ["feed_forward"])
    _check_graph_replays(ff, (4, 64, 256), device)


def test_moe_layer_in_a_captured_graph(device):
    """Routing, group padding, gathered casts, grouped GEMMs and the combine: all group sizes
    stay on the device, so the whole layer replays with routing that differs from step to step."""
    torch.manual_seed(37)
    cfg = MoE.Config(num_experts=8, num_shared_experts=1, top_k=2, hidden_dim=256,
                     score_before_experts=False, score_func="softmax", route_norm=True)
    moe = MoE(cfg, dim=256).to(device).to(torch.bfloat16)
    moe.init_weights(init_std=0.05, buffer_device=device)
    holder = nn.Module()
    holder.moe = moe
    _convert(holder, ["experts"])
    _check_graph_replays(moe, (2, 96, 256), device)


def test_single_linear_captured_after_a_warm_up_on_the_same_static_input(device):
    """The usual recipe, warm-up then capture, on a model whose only cast input is the static
    input itself: the warm-up leaves that tensor's cast in the reuse slot, and the capture must
    not take it."""
    torch.manual_seed(41)
    holder = nn.Module()
    holder.proj = Linear.Config().build(in_features=256, out_features=384)
    holder.to(device).to(torch.bfloat16)
    holder.proj.init_weights(init_std=0.05)
    _convert(holder, ["proj"])
    shape = (4, 64, 256)
    inputs = [torch.randn(shape, device=device, dtype=torch.bfloat16) for _ in range(3)]
    x = torch.zeros(shape, device=device, dtype=torch.bfloat16)
    with torch.no_grad():
        eager = [holder.proj(xi).clone() for xi in inputs]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            holder.proj(x)  # warm-up on the static input, no backward: the reuse slot now holds x's cast
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y = holder.proj(x)
        for rep in range(2):
            for xi, want in zip(inputs, eager):
                x.copy_(xi)
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(y, want), rep
                # eager calls on the same static tensor between replays see its new contents too
                assert torch.equal(holder.proj(x), want)
