"""GPU: the converted modules (F.linear / torch._grouped_mm interception, autograd) vs the oracle."""
import numpy as np
import pytest
import torch
import torch.nn as nn

from oracle import mx_oracle as mo
from tests.helpers import bf16_from_bits, bits_of, randn_bits, rel_l2
from torchtitan_amd.modules import FeedForward, GroupedExperts, Linear, MoE
from torchtitan_amd import ops
from torchtitan_amd.modules import moe as moe_mod
from torchtitan_amd.mx_tensor import MXFP8TrainingWeight
from torchtitan_amd.protocols import ModelConvertersContainer
from torchtitan_amd.quantization.mx import MXFP8Converter

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _f32(bits):
    return mo.bf16_bits_to_f32(bits)


def _convert(model, fqns, recipe="mxfp8_rceil", pad=True, fuse=True, cache=False, norm=False):
    box = ModelConvertersContainer.Config(
        converters=[MXFP8Converter.Config(fqns=fqns, recipe_name=recipe, pad_token_groups_for_grouped_mm=pad,
                                          fuse_swiglu_cast=fuse, cache_weight_casts=cache,
                                          fuse_rmsnorm_cast=norm)]
    ).build(parallel_dims=None, model_compile_enabled=False)
    box.convert(model)
    return box


@pytest.mark.parametrize("recipe,mode", [("mxfp8_rceil", mo.RCEIL), ("mxfp8_floor", mo.FLOOR)])
@pytest.mark.parametrize("M,K,N", [(256, 128, 192), (96, 64, 32), (1000, 256, 320)])
def test_linear_module_three_passes(device, recipe, mode, M, K, N):
    rng = np.random.default_rng(M + K + N)
    x_bits = randn_bits(rng, (M, K), outliers=1e-3)
    w_bits = randn_bits(rng, (N, K), std=0.02)
    dy_bits = randn_bits(rng, (M, N), std=1e-3)
    with torch.device("meta"):
        model = nn.Sequential()
        model.add_module("proj", Linear.Config().build(in_features=K, out_features=N))
    _convert(model, ["proj"], recipe)
    model.to_empty(device=device)
    model.to(torch.bfloat16)
    with torch.no_grad():
        model.proj.weight.copy_(bf16_from_bits(w_bits, device))
    assert isinstance(model.proj.weight, MXFP8TrainingWeight)
    x = bf16_from_bits(x_bits, device).requires_grad_(True)
    y = model(x)
    assert y.dtype == torch.bfloat16 and y.shape == (M, N)
    y.backward(bf16_from_bits(dy_bits, device))
    assert rel_l2(_f32(bits_of(y)), _f32(mo.linear_fwd(x_bits, w_bits, mode))) <= TOL
    # the oracle's wgrad needs M % 32 == 0: pad tokens with zero rows, as the product does
    pad = -M % 32
    xb = np.vstack((x_bits, np.zeros((pad, K), np.uint16)))
    dyb = np.vstack((dy_bits, np.zeros((pad, N), np.uint16)))
    assert rel_l2(_f32(bits_of(x.grad)), _f32(mo.linear_dgrad(dy_bits, w_bits, mode))) <= TOL
    assert rel_l2(_f32(bits_of(model.proj.weight.grad)), _f32(mo.linear_wgrad(dyb, xb, mode))) <= TOL


def test_linear_fp32_master_weights_under_autocast(device):
    torch.manual_seed(0)
    lin = Linear.Config(bias=True).build(in_features=128, out_features=64).to(device)
    lin.init_weights()
    box = nn.Sequential()
    box.add_module("w", lin)
    _convert(box, ["w"])
    x = torch.randn(4, 32, 128, device=device, requires_grad=True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = box(x)
    assert y.dtype == torch.bfloat16 and y.shape == (4, 32, 64)
    y.float().sum().backward()
    assert lin.weight.grad.dtype == torch.float32 and x.grad.dtype == torch.float32
    ref = torch.nn.functional.linear(x.detach(), lin.weight.detach().as_subclass(torch.Tensor), lin.bias.detach())
    assert rel_l2(y.detach().float().cpu().numpy(), ref.float().cpu().numpy()) < 0.05


def test_feed_forward_close_to_bf16_and_trains(device):
    torch.manual_seed(1)
    ff = FeedForward.Config(hidden_dim=512).build(dim=256).to(device).to(torch.bfloat16)
    ff.init_weights(init_std=0.02)
    ref = FeedForward.Config(hidden_dim=512).build(dim=256).to(device).to(torch.bfloat16)
    ref.load_state_dict(ff.state_dict())
    holder = nn.Module()
    holder.feed_forward = ff
    _convert(holder, ["feed_forward"])
    x = torch.randn(2, 128, 256, device=device, dtype=torch.bfloat16)
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = ff(xa), ref(xb)
    ya.float().pow(2).sum().backward()
    yb.float().pow(2).sum().backward()
    assert rel_l2(ya.detach().float().cpu().numpy(), yb.detach().float().cpu().numpy()) < 0.08
    assert rel_l2(xa.grad.float().cpu().numpy(), xb.grad.float().cpu().numpy()) < 0.12
    for n in ("w1", "w2", "w3"):
        ga, gb = getattr(ff, n).weight.grad, getattr(ref, n).weight.grad
        assert rel_l2(ga.float().cpu().numpy(), gb.float().cpu().numpy()) < 0.12
    opt = torch.optim.AdamW(ff.parameters(), lr=1e-3)
    before = ff.w1.weight.detach().clone()
    opt.step()
    assert isinstance(ff.w1.weight, MXFP8TrainingWeight) and not torch.equal(before, ff.w1.weight)


@pytest.mark.parametrize("recipe", ["mxfp8_rceil", "mxfp8_floor"])
@pytest.mark.parametrize("tokens,dim,hidden", [(256, 256, 512), (96, 128, 352)])
def test_feed_forward_fused_gate_matches_separate_ops(device, recipe, tokens, dim, hidden):
    """The SwiGLU block with the gate inside the cast kernel against the same block with silu and
    the product as separate bf16 ops: the output and the weight gradients are bit-identical.  The
    input gradient d(h1) W1 + d(h3) W3 is one GEMM in the fused block where the kernel takes the
    shape (summed in float32, rounded once; `test_pair_gemm_*` pins it against the oracle) against
    two GEMMs and a bf16 add.  The two halves partly cancel, so the separate form's three
    roundings weigh about 3e-3 of the result: rel-L2 <= 5e-3 there, bit-identical where the fused
    block falls back to two GEMMs."""
    torch.manual_seed(7)
    blocks = []
    for fuse in (True, False):
        ff = FeedForward.Config(hidden_dim=hidden).build(dim=dim).to(device).to(torch.bfloat16)
        if blocks:
            ff.load_state_dict(blocks[0].feed_forward.state_dict())
        else:
            ff.init_weights(init_std=0.05)
        holder = nn.Module()
        holder.feed_forward = ff
        _convert(holder, ["feed_forward"], recipe=recipe, fuse=fuse)
        blocks.append(holder)
    x = torch.randn(tokens, dim, device=device, dtype=torch.bfloat16) * 2
    dy = torch.randn(tokens, dim, device=device, dtype=torch.bfloat16)
    outs = []
    for holder in blocks:
        xi = x.clone().requires_grad_(True)
        y = holder.feed_forward(xi)
        y.backward(dy)
        ff = holder.feed_forward
        outs.append([y.detach(), xi.grad, ff.w1.weight.grad, ff.w2.weight.grad, ff.w3.weight.grad])
    for i, (got, want) in enumerate(zip(*outs)):
        if i == 1 and hidden % 128 == 0 and tokens > 128 and dim > 128:
            assert rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy()) <= 5e-3
        else:
            assert torch.equal(got, want), i
    # the fused forward keeps no bf16 gate tensor: the graph node of y is the fused function
    y = blocks[0].feed_forward(x.clone().requires_grad_(True))
    assert type(y.grad_fn).__name__ == "_MXFeedForwardBackward"


def test_feed_forward_fused_with_float32_master_weights(device):
    """float32 parameters, bf16 activations: the fused block casts the weights to bf16 on the
    way in and returns float32 weight gradients, bit-identical to the separate-op form."""
    torch.manual_seed(13)
    blocks = []
    for fuse in (True, False):
        ff = FeedForward.Config(hidden_dim=256).build(dim=128).to(device)
        if blocks:
            ff.load_state_dict(blocks[0].state_dict())
        else:
            ff.init_weights(init_std=0.05)
        holder = nn.Module()
        holder.feed_forward = ff
        _convert(holder, ["feed_forward"], fuse=fuse)
        blocks.append(ff)
    x = torch.randn(96, 128, device=device, dtype=torch.bfloat16)
    dy = torch.randn(96, 128, device=device, dtype=torch.bfloat16)
    outs = []
    for ff in blocks:
        xi = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = ff(xi)
        y.backward(dy)
        assert y.dtype == torch.bfloat16 and ff.w1.weight.grad.dtype == torch.float32
        outs.append([y.detach(), xi.grad, ff.w1.weight.grad, ff.w2.weight.grad, ff.w3.weight.grad])
    for got, want in zip(*outs):
        assert torch.equal(got, want)


@pytest.mark.parametrize("fuse", [True, False])
def test_converted_blocks_under_activation_checkpointing(device, fuse):
    """torch.utils.checkpoint around a converted block (full activation checkpointing, as
    torchtitan applies per layer): the forward is re-run in backward through the same kernels and
    every gradient equals the one without checkpointing."""
    from torch.utils.checkpoint import checkpoint

    torch.manual_seed(17)
    ff = FeedForward.Config(hidden_dim=256).build(dim=128).to(device).to(torch.bfloat16)
    ff.init_weights(init_std=0.05)
    holder = nn.Module()
    holder.feed_forward = ff
    _convert(holder, ["feed_forward"], fuse=fuse)
    x = torch.randn(2, 64, 128, device=device, dtype=torch.bfloat16)
    dy = torch.randn(2, 64, 128, device=device, dtype=torch.bfloat16)
    grads = []
    for use_ckpt in (False, True):
        for p in ff.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        y = checkpoint(ff, xi, use_reentrant=False) if use_ckpt else ff(xi)
        y.backward(dy)
        grads.append([y.detach(), xi.grad] + [p.grad.clone() for p in ff.parameters()])
    for a, b in zip(*grads):
        assert torch.equal(a, b)


@pytest.mark.parametrize("fuse", [True, False])
def test_per_op_checkpoint_policy_can_keep_gemm_outputs(device, fuse, monkeypatch):
    """Selective activation checkpointing by op (the policy shape of
    torchtitan/distributed/activation_checkpoint.py:105-141 over a save list like
    torchtitan/models/llama3/parallelize.py:44-60): with this package's dispatcher ops in the save
    list the three forward GEMMs of a block are not run again in the recomputation (9 GEMM
    launches instead of 12), and every result equals the one without checkpointing."""
    from torch.utils.checkpoint import CheckpointPolicy, checkpoint, create_selective_checkpoint_contexts

    save = ops.op_sac_save_list() | {torch.ops.aten.mm.default}

    def policy(ctx, func, *args, **kwargs):
        return CheckpointPolicy.MUST_SAVE if func in save else CheckpointPolicy.PREFER_RECOMPUTE

    launches = []
    real_call = ops._call
    monkeypatch.setattr(ops, "_call", lambda name, *a: (launches.append(name), real_call(name, *a))[1])

    torch.manual_seed(23)
    ff = FeedForward.Config(hidden_dim=256).build(dim=128).to(device).to(torch.bfloat16)
    ff.init_weights(init_std=0.05)
    holder = nn.Module()
    holder.feed_forward = ff
    _convert(holder, ["feed_forward"], fuse=fuse)
    x = torch.randn(2, 64, 128, device=device, dtype=torch.bfloat16)
    dy = torch.randn(2, 64, 128, device=device, dtype=torch.bfloat16)
    runs = {}
    for how in ("plain", "full", "per_op"):
        for p in ff.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        launches.clear()
        if how == "plain":
            y = ff(xi)
        elif how == "full":
            y = checkpoint(ff, xi, use_reentrant=False)
        else:
            y = checkpoint(ff, xi, use_reentrant=False,
                           context_fn=lambda: create_selective_checkpoint_contexts(policy))
        y.backward(dy)
        # (mx_gemm_nt_ld: the same GEMM on operands whose rows carry the dense linear's pitch)
        runs[how] = (launches.count("mx_gemm_nt") + launches.count("mx_gemm_nt_ld"),
                     [y.detach(), xi.grad] + [p.grad.clone() for p in ff.parameters()])
    assert [runs[h][0] for h in ("plain", "full", "per_op")] == [9, 12, 9]
    for how in ("full", "per_op"):
        for a, b in zip(runs["plain"][1], runs[how][1]):
            assert torch.equal(a, b)


@pytest.mark.parametrize("fuse", [True, False])
def test_per_op_checkpoint_policy_keeps_grouped_gemm_outputs(device, fuse, monkeypatch):
    """As above for the expert block: three forward grouped GEMMs kept, three launches of the 2d3d
    kernel per step fewer than under full checkpointing, results unchanged."""
    from torch.utils.checkpoint import CheckpointPolicy, checkpoint, create_selective_checkpoint_contexts

    save = ops.op_sac_save_list()

    def policy(ctx, func, *args, **kwargs):
        return CheckpointPolicy.MUST_SAVE if func in save else CheckpointPolicy.PREFER_RECOMPUTE

    launches = []
    real_call = ops._call
    # (the form that writes unpadded rows serves one product or, with a second operand set, a sum of two)
    tag = lambda name, a: name + ("_sum_of_two" if name == "mx_grouped_gemm_2d3d_rows_out" and a[6] is not None else "")
    monkeypatch.setattr(ops, "_call", lambda name, *a: (launches.append(tag(name, a)), real_call(name, *a))[1])
    torch.manual_seed(29)
    moe_mod.set_token_group_alignment_size_m(32)
    try:
        counts = torch.tensor([40, 0, 200, 16, 7, 130], device=device)
        ex = GroupedExperts(dim=128, hidden_dim=256, num_experts=6, use_grouped_mm=True).to(device).to(torch.bfloat16)
        ex.init_weights(init_std=0.05)
        holder = nn.Module()
        holder.experts = ex
        _convert(holder, ["experts"], pad=True, fuse=fuse)
        x = torch.randn(int(counts.sum()), 128, device=device, dtype=torch.bfloat16)
        dy = torch.randn(int(counts.sum()), 128, device=device, dtype=torch.bfloat16)
        runs = {}
        for how in ("plain", "full", "per_op"):
            for p in ex.parameters():
                p.grad = None
            xi = x.clone().requires_grad_(True)
            launches.clear()
            if how == "plain":
                y = ex(xi, counts)
            elif how == "full":
                y = checkpoint(ex, xi, counts, use_reentrant=False)
            else:
                y = checkpoint(ex, xi, counts, use_reentrant=False,
                               context_fn=lambda: create_selective_checkpoint_contexts(policy))
            y.backward(dy)
            # grouped 2D x 3D products computed (the launch for h1 and h3 together computes two)
            runs[how] = (launches.count("mx_grouped_gemm_2d3d") + launches.count("mx_grouped_gemm_2d3d_rows_out")
                         + 2 * launches.count("mx_grouped_gemm_2d3d_shared_a"),
                         [y.detach(), xi.grad, ex.w1.grad.clone(), ex.w2.grad.clone(), ex.w3.grad.clone()])
        # forward 3; backward: d(g), and d(x) as two launches or as one of the paired form
        base = 4 if fuse else 6
        assert [runs[h][0] for h in ("plain", "full", "per_op")] == [base, base + 3, base]
        for how in ("full", "per_op"):
            for a, b in zip(runs["plain"][1], runs[how][1]):
                assert torch.equal(a, b)
    finally:
        moe_mod.set_token_group_alignment_size_m(8)


class _NormedBlock(nn.Module):
    """RMSNorm -> three projections sharing the normalised input, and RMSNorm -> SwiGLU block,
    with the norms inside the casts when the converter allows it."""

    def __init__(self, dim, inner, ffn):
        super().__init__()
        mk = lambda i, o: Linear.Config().build(in_features=i, out_features=o)
        self.attention = nn.Module()
        self.attention.wq, self.attention.wk, self.attention.wv = mk(dim, dim), mk(dim, inner), mk(dim, inner)
        self.feed_forward = FeedForward.Config(hidden_dim=ffn).build(dim=dim)
        self.attention_norm = nn.RMSNorm(dim, eps=1e-5)
        self.ffn_norm = nn.RMSNorm(dim, eps=1e-5)

    def forward(self, x):
        from torchtitan_amd.mx_blocks import (feed_forward_fusable, mx_norm_feed_forward, mx_norm_linears,
                                              norm_fusable)

        a, ff = self.attention, self.feed_forward
        qkv_w = (a.wq.weight, a.wk.weight, a.wv.weight)
        if norm_fusable(x, self.attention_norm.weight, *qkv_w):
            q, k, v = mx_norm_linears(x, self.attention_norm.weight, self.attention_norm.eps, qkv_w)
        else:
            h = self.attention_norm(x)
            q, k, v = a.wq(h), a.wk(h), a.wv(h)
        mixed = q + torch.cat((k, v), dim=-1)[..., : q.shape[-1]]      # stands in for attention
        w = (ff.w1.weight, ff.w2.weight, ff.w3.weight)
        if norm_fusable(mixed, self.ffn_norm.weight, w[0], w[2], for_feed_forward=True) and feed_forward_fusable(mixed, *w):
            return mixed + mx_norm_feed_forward(mixed, self.ffn_norm.weight, self.ffn_norm.eps, *w)
        return mixed + ff(self.ffn_norm(mixed))


def test_rms_norm_inside_the_casts_matches_separate_norms(device):
    """Opt-in fusion of the two RMSNorms of a block into the casts that follow them: output and
    all gradients (inputs, seven weights, both norm weights) agree with the separate-norm form:
    to 2e-3 where only the norm differs (the normalised activation moves by one bf16 step at a
    few elements in a million, which can flip an e4m3 code), to 5e-3 where bf16 sums of three
    partial gradients are formed in a different order (dx and the first norm's weight)."""
    torch.manual_seed(19)
    blocks = []
    for norm in (True, False):
        blk = _NormedBlock(256, 128, 512).to(device).to(torch.bfloat16)
        if blocks:
            blk.load_state_dict(blocks[0].state_dict())
        else:
            for m in blk.modules():
                if isinstance(m, nn.Linear):
                    nn.init.normal_(m.weight, std=0.05)
            with torch.no_grad():
                blk.attention_norm.weight.add_(0.1 * torch.randn_like(blk.attention_norm.weight))
                blk.ffn_norm.weight.add_(0.1 * torch.randn_like(blk.ffn_norm.weight))
        _convert(blk, ["attention", "feed_forward"], norm=norm)
        blocks.append(blk)
    x = torch.randn(2, 128, 256, device=device, dtype=torch.bfloat16)
    dy = torch.randn(2, 128, 256, device=device, dtype=torch.bfloat16)
    outs = []
    for blk in blocks:
        xi = x.clone().requires_grad_(True)
        y = blk(xi)
        y.backward(dy)
        outs.append({"y": y.detach(), "dx": xi.grad, **{n: p.grad for n, p in blk.named_parameters()}})
    fused, plain = outs
    assert set(fused) == set(plain) and len(fused) == 2 + 8
    for name in fused:
        assert fused[name] is not None, name
        tol = 5e-3 if name in ("dx", "attention_norm.weight") else 2e-3
        assert rel_l2(fused[name].float().cpu().numpy(), plain[name].float().cpu().numpy()) <= tol, name
    from torchtitan_amd.mx_blocks import norm_fusable
    assert norm_fusable(x, blocks[0].attention_norm.weight, blocks[0].attention.wq.weight)
    assert not norm_fusable(x, blocks[1].attention_norm.weight, blocks[1].attention.wq.weight)


def test_feed_forward_with_only_w2_converted_fuses_the_gate(device):
    """w1 / w3 left in bf16, w2 converted: the gate still runs inside the cast that feeds w2 and
    the block matches the same block built from separate ops bit for bit."""
    torch.manual_seed(11)
    blocks = []
    for fuse in (True, False):
        ff = FeedForward.Config(hidden_dim=384).build(dim=128).to(device).to(torch.bfloat16)
        if blocks:
            ff.load_state_dict(blocks[0].feed_forward.state_dict())
        else:
            ff.init_weights(init_std=0.05)
        holder = nn.Module()
        holder.feed_forward = ff
        _convert(holder, ["feed_forward.w2"], fuse=fuse)
        blocks.append(holder)
    x = torch.randn(4, 40, 128, device=device, dtype=torch.bfloat16)
    dy = torch.randn(4, 40, 128, device=device, dtype=torch.bfloat16)
    outs = []
    for holder in blocks:
        xi = x.clone().requires_grad_(True)
        y = holder.feed_forward(xi)
        y.backward(dy)
        ff = holder.feed_forward
        outs.append([y.detach(), xi.grad, ff.w1.weight.grad, ff.w2.weight.grad, ff.w3.weight.grad])
    for got, want in zip(*outs):
        assert torch.equal(got, want)
    y = blocks[0].feed_forward(x.clone().requires_grad_(True))
    assert type(y.grad_fn).__name__ == "_MXSwiGLULinearBackward"


def test_feed_forward_fused_with_frozen_parts(device):
    """Only some inputs of the fused block require gradients."""
    torch.manual_seed(12)
    ff = FeedForward.Config(hidden_dim=256).build(dim=128).to(device).to(torch.bfloat16)
    ff.init_weights(init_std=0.05)
    ref = FeedForward.Config(hidden_dim=256).build(dim=128).to(device).to(torch.bfloat16)
    ref.load_state_dict(ff.state_dict())
    for m, fuse in ((ff, True), (ref, False)):
        holder = nn.Module()
        holder.feed_forward = m
        _convert(holder, ["feed_forward"], fuse=fuse)
        m.w1.weight.requires_grad_(False)
    x = torch.randn(64, 128, device=device, dtype=torch.bfloat16)
    dy = torch.randn(64, 128, device=device, dtype=torch.bfloat16)
    ff(x).backward(dy)   # x needs no gradient
    ref(x).backward(dy)
    assert ff.w1.weight.grad is None
    assert torch.equal(ff.w2.weight.grad, ref.w2.weight.grad) and torch.equal(ff.w3.weight.grad, ref.w3.weight.grad)
    for m in (ff, ref):
        for p in m.parameters():
            p.requires_grad_(False)
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ff(xa).backward(dy)
    ref(xb).backward(dy)
    assert torch.equal(xa.grad, xb.grad)


@pytest.mark.parametrize("pad,align", [(True, 8), (False, 32)])
@pytest.mark.parametrize("dim,hidden", [(128, 64), (256, 128)])
def test_grouped_experts_module(device, pad, align, dim, hidden):
    """torch._grouped_mm on converted 3-D weights, forward and backward, vs per-expert oracle.

    With both dims multiples of 128 the wrapper pads groups to 32 rows (the token axis to 128) and
    the persistent kernels run; otherwise the general ones.  The results must not depend on it."""
    rng = np.random.default_rng(17 + align + dim)
    E = 4
    counts = np.array([40, 0, 200, 16]) if pad else np.array([64, 0, 96, 32])
    T = int(counts.sum())
    x_bits = randn_bits(rng, (T, dim))
    w_bits = randn_bits(rng, (E, hidden, dim), std=0.05)
    dy_bits = randn_bits(rng, (T, hidden), std=1e-2)
    w = nn.Parameter(bf16_from_bits(w_bits, device))
    holder = nn.Module()
    holder.experts = nn.Module()
    holder.experts.w1 = w
    _convert(holder, ["experts"], pad=pad)
    w = holder.experts.w1
    assert isinstance(w, MXFP8TrainingWeight)
    x = bf16_from_bits(x_bits, device).requires_grad_(True)
    offs = torch.tensor(np.cumsum(counts), dtype=torch.int32, device=device)
    y = torch._grouped_mm(x, w.bfloat16().transpose(-2, -1), offs=offs)
    y.backward(bf16_from_bits(dy_bits, device))
    ref = mo.grouped_fwd(x_bits, w_bits, np.cumsum(counts), mo.RCEIL)
    assert rel_l2(_f32(bits_of(y)), _f32(ref)) <= TOL
    ref = mo.grouped_dgrad(dy_bits, w_bits, np.cumsum(counts), mo.RCEIL)
    assert rel_l2(_f32(bits_of(x.grad)), _f32(ref)) <= TOL
    # wgrad: every group zero-padded to a multiple of 32 tokens
    xs, dys, sizes = [], [], []
    lo = 0
    for c in counts:
        p = max(-(-c // 32) * 32, 32) if pad else c
        xs.append(np.vstack((x_bits[lo:lo + c], np.zeros((p - c, dim), np.uint16))))
        dys.append(np.vstack((dy_bits[lo:lo + c], np.zeros((p - c, hidden), np.uint16))))
        sizes.append(p)
        lo += c
    ref = mo.grouped_wgrad(np.vstack(dys), np.vstack(xs), np.cumsum(sizes), mo.RCEIL)
    got = bits_of(w.grad)
    for g, c in enumerate(counts):
        if c == 0:
            assert np.all(_f32(got[g]) == 0)
        else:
            assert rel_l2(_f32(got[g]), _f32(ref[g])) <= TOL, g


def test_grouped_experts_swiglu_block(device):
    """GroupedExperts.forward (pad wrapper + three grouped GEMMs) close to its own bf16 loop."""
    torch.manual_seed(3)
    moe_mod.set_token_group_alignment_size_m(32)
    try:
        ex = GroupedExperts(dim=128, hidden_dim=64, num_experts=8, use_grouped_mm=True).to(device).to(torch.bfloat16)
        ex.init_weights(init_std=0.05)
        loop = GroupedExperts(dim=128, hidden_dim=64, num_experts=8, use_grouped_mm=False).to(device).to(torch.bfloat16)
        loop.load_state_dict(ex.state_dict())
        holder = nn.Module()
        holder.experts = ex
        _convert(holder, ["experts"], pad=False)
        counts = torch.tensor([5, 0, 33, 64, 1, 17, 0, 40], device=device)
        x = torch.randn(int(counts.sum()), 128, device=device, dtype=torch.bfloat16)
        ya = ex(x, counts)
        yb = loop(x, counts)
        assert ya.shape == yb.shape
        assert rel_l2(ya.detach().float().cpu().numpy(), yb.detach().float().cpu().numpy()) < 0.1
    finally:
        moe_mod.set_token_group_alignment_size_m(8)


@pytest.mark.parametrize("pad,align", [(True, 8), (False, 32)])
@pytest.mark.parametrize("dim,hidden", [(128, 64), (256, 128)])
def test_grouped_experts_fused_block_matches_separate_ops(device, pad, align, dim, hidden):
    """The expert block as one fused function (one padding pass, gate inside the casts) against
    three converted grouped GEMMs around separate bf16 silu / product ops: bit-identical output
    and weight gradients, on the persistent kernels (pad on, dims % 128) and on the general ones;
    the input gradient (float32 sum of both halves inside one grouped GEMM on the persistent
    kernel) within rel-L2 5e-3 of the separate form's bf16 sum of two rounded halves that partly
    cancel."""
    torch.manual_seed(21)
    moe_mod.set_token_group_alignment_size_m(align)
    try:
        counts = torch.tensor([40, 0, 200, 16, 7, 130] if pad else [64, 0, 96, 32, 32, 160], device=device)
        blocks = []
        for fuse in (True, False):
            ex = GroupedExperts(dim=dim, hidden_dim=hidden, num_experts=6, use_grouped_mm=True).to(device).to(torch.bfloat16)
            if blocks:
                ex.load_state_dict(blocks[0].state_dict())
            else:
                ex.init_weights(init_std=0.05)
            holder = nn.Module()
            holder.experts = ex
            _convert(holder, ["experts"], pad=pad, fuse=fuse)
            blocks.append(ex)
        x = torch.randn(int(counts.sum()), dim, device=device, dtype=torch.bfloat16)
        dy = torch.randn(int(counts.sum()), dim, device=device, dtype=torch.bfloat16)
        outs = []
        for ex in blocks:
            xi = x.clone().requires_grad_(True)
            y = ex(xi, counts)
            y.backward(dy)
            outs.append([y.detach(), xi.grad, ex.w1.grad, ex.w2.grad, ex.w3.grad])
        for i, (got, want) in enumerate(zip(*outs)):
            if i == 1:  # dx: one grouped GEMM over both halves (one rounding) against two and an add
                assert rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy()) <= 5e-3
            else:
                assert torch.equal(got, want), i
        assert not torch.isnan(outs[0][0]).any() and outs[0][2].abs().sum() > 0
        from torchtitan_amd.mx_blocks import grouped_feed_forward_fusable as fusable
        assert fusable(x, blocks[0].w1, blocks[0].w2, blocks[0].w3)
        assert not fusable(x, blocks[1].w1, blocks[1].w2, blocks[1].w3)
    finally:
        moe_mod.set_token_group_alignment_size_m(8)


@pytest.mark.parametrize("score_before", [True, False])
@pytest.mark.parametrize("dim,hidden,experts,top_k", [(128, 64, 8, 2), (256, 128, 16, 4)])
def test_moe_layer_fused_routing_matches_torch_ops(device, score_before, dim, hidden, experts, top_k):
    """MoE layer with gather + score + experts + combine as one fused function against the same
    layer built from torch's gather / scatter / bmm around the converted experts.  Expert weight
    gradients are bit-identical (the experts see bit-identical inputs and output gradients); the
    output, dx and the router's gradient differ only by float32 summation order over top_k and
    over the row dot products: rel-L2 <= 2e-3 (bf16 rounding of a differently ordered sum); 5e-3
    for dx and the router's gradient, where the fused form also sums the two halves of the
    experts' input gradient in float32 inside one grouped GEMM and the other rounds each half
    (halves that partly cancel, so their roundings weigh about 3e-3 of the sum)."""
    torch.manual_seed(5)
    layers = []
    for fuse in (True, False):
        cfg = MoE.Config(num_experts=experts, num_shared_experts=1, top_k=top_k, hidden_dim=hidden,
                         score_before_experts=score_before, score_func="softmax", route_norm=True)
        moe = MoE(cfg, dim=dim).to(device).to(torch.bfloat16)
        if layers:
            moe.load_state_dict(layers[0].state_dict())
        else:
            moe.init_weights(init_std=0.05, buffer_device=device)
        holder = nn.Module()
        holder.moe = moe
        _convert(holder, ["experts"], fuse=fuse)   # shared experts and the router stay in bf16
        layers.append(moe)
    x = torch.randn(2, 96, dim, device=device, dtype=torch.bfloat16)
    dy = torch.randn(2, 96, dim, device=device, dtype=torch.bfloat16)
    outs = []
    for moe in layers:
        xi = x.clone().requires_grad_(True)
        y = moe(xi)
        y.backward(dy)
        outs.append(dict(y=y.detach(), dx=xi.grad, gate=moe.router.gate.weight.grad, w1=moe.experts.w1.grad,
                         w2=moe.experts.w2.grad, w3=moe.experts.w3.grad, counts=moe.tokens_per_expert.clone()))
    a, b = outs
    assert torch.equal(a["counts"], b["counts"]) and a["counts"].sum() == 2 * 96 * top_k
    for name in ("w1", "w2", "w3"):
        assert torch.equal(a[name], b[name]), name
    for name, tol in (("y", 2e-3), ("dx", 5e-3), ("gate", 5e-3)):
        assert rel_l2(a[name].float().cpu().numpy(), b[name].float().cpu().numpy()) <= tol, name


def test_weight_cast_cache_and_mxfp8_hand_over(device):
    """cache_weight_casts: same results as without; the casts are reused until the weight is
    updated in place; the post-optimizer hook refreshes them; the exported MXFP8 state dict
    dequantizes to exactly what the GEMMs multiply by and takes 33/64 of the bf16 bytes."""
    from torchtitan_amd import mx_tensor, ops
    from torchtitan_amd.quantization.mx import export_mxfp8_state_dict, load_mxfp8_state_dict

    torch.manual_seed(9)
    mx_tensor._weight_cache.clear()
    blocks, boxes = [], []
    for cache in (True, False):
        ff = FeedForward.Config(hidden_dim=256).build(dim=128).to(device).to(torch.bfloat16)
        if blocks:
            ff.load_state_dict(blocks[0].state_dict())
        else:
            ff.init_weights(init_std=0.05)
        holder = nn.Module()
        holder.feed_forward = ff
        boxes.append(_convert(holder, ["feed_forward"], cache=cache))
        blocks.append(ff)
    cached, plain = blocks
    x = torch.randn(64, 128, device=device, dtype=torch.bfloat16).requires_grad_(True)
    calls = []
    real = ops.to_mx_dim0_dim1
    ops.to_mx_dim0_dim1 = lambda t, *a, **k: (calls.append(tuple(t.shape)), real(t, *a, **k))[1]
    try:
        for step in range(2):
            for micro in range(2):          # two micro-batches per optimizer step
                ya, yb = cached(x), plain(x)
                assert torch.equal(ya, yb)
                ya.sum().backward()
                yb.sum().backward()
            for a, b in zip(cached.parameters(), plain.parameters()):
                assert torch.equal(a.grad, b.grad)
            w_casts = [c for c in calls if c in ((256, 128), (128, 256))]
            # plain: 3 weights x 2 micro-batches; cached: 3 weights once in the first step, none
            # after the hook has cast them
            assert len(w_casts) == (9 if step == 0 else 6), (step, w_casts)
            calls.clear()
            with torch.no_grad():
                for m in (cached, plain):
                    for p in m.parameters():
                        p.add_(p.grad, alpha=-0.1)   # the optimizer's in-place update
                        p.grad = None
            holder = nn.Module()
            holder.feed_forward = cached
            boxes[0].post_optimizer_hook(holder)
            assert len([c for c in calls if c in ((256, 128), (128, 256))]) == 3  # cast once, in the hook
            calls.clear()
        ya, yb = cached(x), plain(x)
        assert torch.equal(ya, yb)
        assert len([c for c in calls if c in ((256, 128), (128, 256))]) == 3  # only the uncached block casts
    finally:
        ops.to_mx_dim0_dim1 = real
    payload = export_mxfp8_state_dict(cached)
    sd = cached.state_dict()
    assert set(payload) == set(sd)
    entry = payload["w1.weight"]
    assert entry["codes"].shape == (256, 128) and entry["scales"].shape == (256, 4)
    sent = sum(v["codes"].numel() + v["scales"].numel() for v in payload.values())
    assert sent * 64 == sum(t.numel() * 2 for t in sd.values()) * 33
    back = load_mxfp8_state_dict(payload)
    q = ops.to_mx_dim0(sd["w1.weight"].as_subclass(torch.Tensor), "rceil", ops.MX_SCALES_ROWMAJOR)
    assert torch.equal(back["w1.weight"], ops.mx_dequant(q))
    assert rel_l2(back["w2.weight"].float().cpu().numpy(), sd["w2.weight"].float().cpu().numpy()) < 0.04
    mx_tensor._weight_cache.clear()


class _MiniDecoderBlock(nn.Module):
    """Llama-style block in small: RMSNorm, GQA attention with RoPE-free SDPA in bf16, SwiGLU FFN.
    The seven linears are the `Linear` modules the converter selects by FQN."""

    def __init__(self, dim, heads, kv_heads, ffn):
        super().__init__()
        self.heads, self.kv_heads, self.hd = heads, kv_heads, dim // heads
        self.attention = nn.Module()
        mk = lambda i, o: Linear.Config().build(in_features=i, out_features=o)
        self.attention.wq = mk(dim, dim)
        self.attention.wk = mk(dim, kv_heads * self.hd)
        self.attention.wv = mk(dim, kv_heads * self.hd)
        self.attention.wo = mk(dim, dim)
        self.feed_forward = FeedForward.Config(hidden_dim=ffn).build(dim=dim)
        self.n1 = nn.RMSNorm(dim, eps=1e-5)
        self.n2 = nn.RMSNorm(dim, eps=1e-5)

    def forward(self, x):
        B, S, D = x.shape
        h = self.n1(x)
        q = self.attention.wq(h).view(B, S, self.heads, self.hd).transpose(1, 2)
        k = self.attention.wk(h).view(B, S, self.kv_heads, self.hd).transpose(1, 2)
        v = self.attention.wv(h).view(B, S, self.kv_heads, self.hd).transpose(1, 2)
        rep = self.heads // self.kv_heads
        k, v = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)
        a = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
        x = x + self.attention.wo(a.transpose(1, 2).reshape(B, S, D))
        return x + self.feed_forward(self.n2(x))


def test_decoder_block_with_all_seven_linears_converted(device):
    """The converter drops into a whole block: same module tree, every linear selected by FQN,
    output and gradients close to the unconverted bf16 block, parameters still trainable."""
    torch.manual_seed(7)
    blk = _MiniDecoderBlock(256, 4, 2, 512).to(device).to(torch.bfloat16)
    for m in blk.modules():
        if isinstance(m, nn.Linear):
            nn.init.normal_(m.weight, std=0.02)
    ref = _MiniDecoderBlock(256, 4, 2, 512).to(device).to(torch.bfloat16)
    ref.load_state_dict(blk.state_dict())
    _convert(blk, ["attention", "feed_forward"])
    wrapped = [n for n, p in blk.named_parameters() if isinstance(p, MXFP8TrainingWeight)]
    assert len(wrapped) == 7
    x = torch.randn(1, 256, 256, device=device, dtype=torch.bfloat16)
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    ya, yb = blk(xa), ref(xb)
    ya.float().pow(2).mean().backward()
    yb.float().pow(2).mean().backward()
    assert rel_l2(ya.detach().float().cpu().numpy(), yb.detach().float().cpu().numpy()) < 0.05
    assert rel_l2(xa.grad.float().cpu().numpy(), xb.grad.float().cpu().numpy()) < 0.1
    for (n, pa), (_, pb) in zip(blk.named_parameters(), ref.named_parameters()):
        if pa.ndim == 2:
            assert rel_l2(pa.grad.float().cpu().numpy(), pb.grad.float().cpu().numpy()) < 0.15, n


@pytest.mark.parametrize("fuse", [False, True])
def test_decoder_block_under_torch_compile_equals_eager(device, fuse):
    """The block wrapped as the reference wraps its transformer blocks
    (torchtitan/models/llama3/parallelize.py:271-284: ``torch.compile(block, fullgraph=True)``):
    every converted linear -- with the gate fusion on, the whole SwiGLU block -- enters the graph
    as one opaque operator, forward and backward run without a graph break, and output and all
    gradients equal the eager run of the same configuration bit for bit.  The backend replays the
    traced graph op by op, so no code generator for the glue ops is involved."""
    import torch._dynamo

    torch.manual_seed(17)
    blk = _MiniDecoderBlock(256, 4, 2, 512).to(device).to(torch.bfloat16)
    for m in blk.modules():
        if isinstance(m, nn.Linear):
            nn.init.normal_(m.weight, std=0.02)
    _convert(blk, ["attention", "feed_forward"], fuse=fuse)
    x = torch.randn(2, 128, 256, device=device, dtype=torch.bfloat16)
    dy = torch.randn_like(x) * 1e-2

    def run(fn):
        for p in blk.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        y = fn(xi)
        y.backward(dy)
        return [y.detach().clone(), xi.grad.clone()] + [p.grad.clone() for p in blk.parameters()]

    want = run(blk)
    torch._dynamo.reset()
    compiled_blk = torch.compile(blk, backend="aot_eager", fullgraph=True)
    launches = []
    real_call = ops._call
    ops._call = lambda name, *a: (launches.append(name), real_call(name, *a))[1]
    try:
        got = run(compiled_blk)
    finally:
        ops._call = real_call
    # with the fusion on the compiled block runs the gate kernels, not separate silu / product ops
    assert ("mx_swiglu_cast_dim0_dim1_ld" in launches) == fuse and ("mx_swiglu_bwd_cast_dim0_dim1_ld" in launches) == fuse
    again = run(compiled_blk)  # the second call reuses the compiled graph
    assert len(got) == len(want)
    for g, a, w in zip(got, again, want):
        assert torch.equal(g, w) and torch.equal(a, w)
    torch._dynamo.reset()


@pytest.mark.parametrize("fuse", [False, True])
@pytest.mark.parametrize("pad,align", [(True, 8), (False, 32)])
@pytest.mark.parametrize("dim,hidden", [(128, 256), (96, 160)])
def test_grouped_experts_under_torch_compile_equal_eager(device, pad, align, dim, hidden, fuse):
    """The expert block compiled as one graph (the reference compiles MoE blocks as well): each
    converted grouped GEMM is one opaque operator that holds the padding plan, the casts and the
    grouped kernels of the eager path, so output and all gradients equal the eager run bit for
    bit (gate fusion off on the eager side: the same unfused sequence).  With experts that pad
    their own groups the compiled block leaves the outer padding wrapper out; rows of real
    tokens do not depend on where padding rows sit."""
    import torch._dynamo

    torch.manual_seed(23)
    moe_mod.set_token_group_alignment_size_m(align)
    try:
        ex = GroupedExperts(dim=dim, hidden_dim=hidden, num_experts=6, use_grouped_mm=True).to(device).to(torch.bfloat16)
        ex.init_weights(init_std=0.05)
        holder = nn.Module()
        holder.experts = ex
        _convert(holder, ["experts"], pad=pad, fuse=fuse)
        counts = torch.tensor([5, 0, 33, 64, 1, 41], device=device)
        x = torch.randn(int(counts.sum()), dim, device=device, dtype=torch.bfloat16)
        dy = torch.randn_like(x) * 1e-2

        def run(fn):
            for p in ex.parameters():
                p.grad = None
            xi = x.clone().requires_grad_(True)
            y = fn(xi, counts)
            y.backward(dy)
            return [y.detach().clone(), xi.grad.clone()] + [p.grad.clone() for p in ex.parameters()]

        want = run(ex)
        torch._dynamo.reset()
        compiled_ex = torch.compile(ex, backend="aot_eager", fullgraph=True)
        got = run(compiled_ex)
        again = run(compiled_ex)
        for g, a, w in zip(got, again, want):
            assert torch.equal(g, w) and torch.equal(a, w)
    finally:
        moe_mod.set_token_group_alignment_size_m(8)
        torch._dynamo.reset()


@pytest.mark.parametrize("fuse", [False, True])
@pytest.mark.parametrize("score_before", [True, False])
def test_moe_layer_under_torch_compile_equals_eager(device, fuse, score_before):
    """Router, reordering, converted experts, shared experts and the combine as one compiled
    graph without a break; bit-identical to the eager layer of the same configuration (fused: the
    routed half is one operator with gather, score multiply and combine inside its kernels)."""
    import torch._dynamo

    torch.manual_seed(29)
    cfg = MoE.Config(num_experts=8, num_shared_experts=1, top_k=2, hidden_dim=128,
                     score_before_experts=score_before, score_func="softmax", route_norm=True)
    moe = MoE(cfg, dim=256).to(device).to(torch.bfloat16)
    moe.init_weights(init_std=0.05, buffer_device=device)
    holder = nn.Module()
    holder.moe = moe
    _convert(holder, ["experts"], fuse=fuse)
    x = torch.randn(2, 96, 256, device=device, dtype=torch.bfloat16)
    dy = torch.randn_like(x)

    def run(fn):
        for p in moe.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        y = fn(xi)
        y.backward(dy)
        return [y.detach().clone(), xi.grad.clone()] + [p.grad.clone() for p in moe.parameters()]

    try:
        want = run(moe)
        torch._dynamo.reset()
        compiled_moe = torch.compile(moe, backend="aot_eager", fullgraph=True)
        got = run(compiled_moe)
        assert len(got) == len(want)
        for g, w in zip(got, want):
            assert torch.equal(g, w)
    finally:
        torch._dynamo.reset()


def test_norm_inside_the_feed_forward_cast_under_torch_compile_equals_eager(device):
    """RMSNorm + SwiGLU block with the norm inside the cast (opt-in), compiled as one graph: the
    block is one operator whose backward also returns the norm weight's gradient; bit-identical
    to the eager function."""
    import torch._dynamo
    from torchtitan_amd.mx_blocks import feed_forward_fusable, mx_norm_feed_forward, norm_fusable

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.feed_forward = FeedForward.Config(hidden_dim=512).build(dim=256)
            self.ffn_norm = nn.RMSNorm(256, eps=1e-5)

        def forward(self, x):
            w = (self.feed_forward.w1.weight, self.feed_forward.w2.weight, self.feed_forward.w3.weight)
            assert norm_fusable(x, self.ffn_norm.weight, w[0], w[2], for_feed_forward=True) and feed_forward_fusable(x, *w)
            return x + mx_norm_feed_forward(x, self.ffn_norm.weight, self.ffn_norm.eps, *w)

    torch.manual_seed(37)
    blk = Block().to(device).to(torch.bfloat16)
    for lin in (blk.feed_forward.w1, blk.feed_forward.w2, blk.feed_forward.w3):
        nn.init.normal_(lin.weight, std=0.05)
    with torch.no_grad():
        blk.ffn_norm.weight.add_(0.1 * torch.randn_like(blk.ffn_norm.weight))
    _convert(blk, ["feed_forward"], norm=True)
    x = torch.randn(2, 64, 256, device=device, dtype=torch.bfloat16)
    dy = torch.randn_like(x)

    def run(fn):
        for p in blk.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        y = fn(xi)
        y.backward(dy)
        return [y.detach().clone(), xi.grad.clone()] + [p.grad.clone() for p in blk.parameters()]

    try:
        want = run(blk)
        torch._dynamo.reset()
        got = run(torch.compile(blk, backend="aot_eager", fullgraph=True))
        assert len(got) == len(want) == 2 + 4
        for g, w in zip(got, want):
            assert torch.equal(g, w)
    finally:
        torch._dynamo.reset()


def test_compiled_block_without_gradients_runs_the_row_wise_casts_only(device):
    """Under no_grad the traced operators leave the column-wise casts out (nothing is kept for a
    backward) and the output equals the eager one."""
    import torch._dynamo

    torch.manual_seed(41)
    ff = FeedForward.Config(hidden_dim=512).build(dim=256).to(device).to(torch.bfloat16)
    for lin in (ff.w1, ff.w2, ff.w3):
        nn.init.normal_(lin.weight, std=0.05)
    holder = nn.Module()
    holder.ff = ff
    _convert(holder, ["ff"], fuse=False)
    x = torch.randn(256, 256, device=device, dtype=torch.bfloat16)
    launches = []
    real_call = ops._call
    try:
        with torch.no_grad():
            want = ff(x)
            torch._dynamo.reset()
            fn = torch.compile(ff, backend="aot_eager", fullgraph=True)
            ops._call = lambda name, *a: (launches.append(name), real_call(name, *a))[1]
            got = fn(x)
        assert torch.equal(got, want)
        assert launches.count("mx_cast_dim0") == 6 and "mx_cast_dim0_dim1" not in launches and "mx_cast_dim1" not in launches
    finally:
        ops._call = real_call
        torch._dynamo.reset()


def test_feed_forward_under_the_inductor_backend_close_to_eager(device):
    """The reference's default ``torch.compile`` backend generates code for the glue between the
    converted linears (silu, the product); the MXFP8 linears stay the opaque operators.  The
    generated glue keeps float32 between silu and the product where eager rounds to bf16, so
    the comparison is a tolerance, not equality: a gate value that lands on the other side of a
    bf16 rounding step can land on the other side of an e4m3 step (1/16 to 1/8 of the value) in
    the down projection's cast, which moves the output by about one percent in rel-L2.  Bound:
    3e-2 for the output and every gradient (measured 1.2e-2; the bit-identical comparison is the
    aot_eager test above)."""
    import torch._dynamo

    pytest.importorskip("triton")
    torch.manual_seed(31)
    ff = FeedForward.Config(hidden_dim=512).build(dim=256).to(device).to(torch.bfloat16)
    for lin in (ff.w1, ff.w2, ff.w3):
        nn.init.normal_(lin.weight, std=0.02)
    holder = nn.Module()
    holder.ff = ff
    _convert(holder, ["ff"], fuse=False)
    x = torch.randn(256, 256, device=device, dtype=torch.bfloat16)
    dy = torch.randn_like(x) * 1e-2

    def run(fn):
        for p in ff.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        y = fn(xi)
        y.backward(dy)
        return [y.detach().float(), xi.grad.float()] + [p.grad.float() for p in ff.parameters()]

    try:
        want = run(ff)
        torch._dynamo.reset()
        got = run(torch.compile(ff, fullgraph=True))
        for g, w in zip(got, want):
            assert rel_l2(g.cpu().numpy(), w.cpu().numpy()) <= 3e-2
    finally:
        torch._dynamo.reset()
