"""GPU: the two multi-linear benchmark configurations at their full sizes.

* One Llama-3-8B decoder block (torchtitan/models/llama3/__init__.py:116-144): dim 4096, 32 heads /
  8 KV heads, FFN 14336, batch 1 x seq 8192: the seven linears' forward, dgrad and wgrad through
  converted modules, and the whole block.
* One layer of the 1.7B Qwen3-style policy (torchtitan/models/qwen3/__init__.py:120-150): dim 2048,
  16 heads / 8 KV heads of 128, FFN 6144, over the 147 456 packed tokens of a policy step, then
  the MXFP8 hand-over of a 28-layer stack of those weights, and the token log-probabilities at the
  real vocabulary over more rows than one backward launch covers; and the policy step composed:
  packed sequences of uneven lengths through two such layers and the language-model head into the
  policy-gradient loss (torchtitan/experiments/rl/unified/actors/utils.py:56-147), backward, an
  optimizer step and the hand-over.

No CPU pass can follow these sizes, so each result is checked three ways: (1) row blocks of the
output equal the same kernels run on the slice alone, bit for bit (every row of a cast or a GEMM
depends on that row only); (2) 64 x 96 corners of every output, at the origin and at the far end,
against the oracle run on the raw bf16 inputs of that corner (casts and GEMM together, rel-L2 <=
1e-3); (3) the whole block on a token slice against the same block with every linear replaced by
the oracle's (causal attention: the first tokens do not see the rest).
"""
import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import c_oracle as co
from oracle import mx_oracle as mo
from tests.helpers import bf16_from_bits, bits_of, rel_l2
from torchtitan_amd import _lib, ops
from torchtitan_amd.modules import FeedForward, Linear
from torchtitan_amd.mx_blocks import feed_forward_fusable, mx_norm_feed_forward, mx_norm_linears, norm_fusable
from torchtitan_amd.mx_tensor import MXFP8TrainingWeight
from torchtitan_amd.protocols import ModelConvertersContainer
from torchtitan_amd.quantization.mx import MXFP8Converter, export_mxfp8_state_dict

pytestmark = pytest.mark.gpu

TOL = 1e-3  # rel-L2 of a GEMM output against the emulated MX matmul, both rounded to bf16


def _f32(bits):
    return mo.bf16_bits_to_f32(bits)


def _convert(model, fqns, **extra):
    ModelConvertersContainer.Config(
        converters=[MXFP8Converter.Config(fqns=fqns, recipe_name="mxfp8_rceil", **extra)]
    ).build(parallel_dims=None, model_compile_enabled=False).convert(model)


def _oracle_matmul(a_codes, a_scales, b_codes, b_scales):
    """bf16 bits of deq(a) deq(b)^T: exact dequantisation, float32 BLAS accumulation."""
    return mo.f32_to_bf16_bits(co.dequant(a_codes, a_scales) @ co.dequant(b_codes, b_scales).T)


def _corner_checks(x, w, dy, y, dx, dw, corners):
    """Oracle on the raw inputs of 64 x 96 corners of Y = X W^T, dX = dY W, dW = dY^T X (RCEIL)."""
    mode = mo.RCEIL
    M, N = dy.shape
    K = x.shape[1]
    for far in corners:
        r = slice(M - 64, M) if far else slice(0, 64)
        # forward: rows r of X against the last / first 96 rows of W
        c = slice(N - 96, N) if far else slice(0, 96)
        ref = _oracle_matmul(*co.cast_dim0(bits_of(x[r]), mode), *co.cast_dim0(bits_of(w[c]), mode))
        assert rel_l2(_f32(bits_of(y[r, c])), _f32(ref)) <= TOL, ("fwd", far)
        # dgrad: rows r of dY against 96 columns of W, blocks along N
        c = slice(K - 96, K) if far else slice(0, 96)
        ref = _oracle_matmul(*co.cast_dim0(bits_of(dy[r]), mode), *co.cast_dim1(bits_of(w[:, c]), mode))
        assert rel_l2(_f32(bits_of(dx[r, c])), _f32(ref)) <= TOL, ("dgrad", far)
        # wgrad: 64 columns of dY against 96 columns of X, blocks down all M tokens
        rn = slice(N - 64, N) if far else slice(0, 64)
        ref = _oracle_matmul(*co.cast_dim1(bits_of(dy[:, rn]), mode), *co.cast_dim1(bits_of(x[:, c]), mode))
        assert rel_l2(_f32(bits_of(dw[rn, c])), _f32(ref)) <= TOL, ("wgrad", far)


def _one_linear_at_size(device, M, K, N, seed, slice_rows=512):
    """Forward + backward of a converted Linear K -> N over M tokens, checked by (1) and (2)."""
    torch.manual_seed(seed)
    holder = nn.Module()
    holder.proj = Linear.Config().build(in_features=K, out_features=N)
    _convert(holder, ["proj"])
    holder.to(device).to(torch.bfloat16)
    lin = holder.proj
    assert isinstance(lin.weight, MXFP8TrainingWeight)
    with torch.no_grad():
        lin.weight.normal_(0.0, 0.02)
    x = torch.randn(M, K, device=device, dtype=torch.bfloat16).requires_grad_(True)
    dy = torch.randn(M, N, device=device, dtype=torch.bfloat16) * 1e-3
    y = lin(x)
    y.backward(dy)
    dx, dw = x.grad, lin.weight.grad
    w = lin.weight.detach().as_subclass(torch.Tensor)
    assert y.shape == (M, N) and dx.shape == (M, K) and dw.shape == (N, K)
    assert torch.isfinite(y).all() and torch.isfinite(dx).all() and torch.isfinite(dw).all()
    # (1) blocks of rows from the start, an odd place in the middle and the very end: the same
    # kernels on the slice alone (the persistent GEMM kernel for the slice too, so that both
    # sides sum in the same order)
    lib = _lib.load()
    lib.mx_debug_force_kernel(3)
    try:
        for r0 in (0, (M // 2 // 32) * 32 - 96, M - slice_rows):
            rows = slice(r0, r0 + slice_rows)
            xs = x.detach()[rows].clone().requires_grad_(True)
            ys = lin(xs)
            (dxs,) = torch.autograd.grad(ys, [xs], dy[rows].contiguous())  # leaves weight.grad alone
            assert torch.equal(ys, y[rows]), ("fwd rows", r0)
            assert torch.equal(dxs, dx[rows]), ("dgrad rows", r0)
    finally:
        lib.mx_debug_force_kernel(0)
    # (2)
    _corner_checks(x.detach(), w, dy, y.detach(), dx, dw, corners=(False, True))
    return x.detach(), w, dy, dw


LLAMA3_8B_LINEARS = {  # name: (in, out) at dim 4096, 32 heads / 8 KV heads of 128, FFN 14336
    "wq_wo": (4096, 4096), "wk_wv": (4096, 1024), "w1_w3": (4096, 14336), "w2": (14336, 4096)}


@pytest.mark.parametrize("name", list(LLAMA3_8B_LINEARS))
def test_llama3_8b_block_linears_at_seq_8192(device, name):
    K, N = LLAMA3_8B_LINEARS[name]
    _one_linear_at_size(device, 8192, K, N, seed=len(name) + K + N)


# ---- the whole block ---------------------------------------------------------------------------
class _Attention(nn.Module):
    def __init__(self, dim, heads, kv_heads, qk_norm_eps=None):
        super().__init__()
        self.dim, self.heads, self.kv_heads, self.hd = dim, heads, kv_heads, dim // heads
        mk = lambda i, o: Linear.Config().build(in_features=i, out_features=o)
        self.wq, self.wo = mk(dim, dim), mk(dim, dim)
        self.wk, self.wv = mk(dim, kv_heads * self.hd), mk(dim, kv_heads * self.hd)
        # Qwen3 normalises q and k per head in front of the rotation (torchtitan/models/qwen3/__init__.py:120-150)
        self.q_norm = nn.RMSNorm(self.hd, eps=qk_norm_eps) if qk_norm_eps is not None else None
        self.k_norm = nn.RMSNorm(self.hd, eps=qk_norm_eps) if qk_norm_eps is not None else None

    def qkv(self, x, norm):
        qkv_w = (self.wq.weight, self.wk.weight, self.wv.weight)
        if norm_fusable(x, norm.weight, *qkv_w):  # opt-in: the norm inside the cast of x
            return mx_norm_linears(x, norm.weight, norm.eps, qkv_w)
        h = norm(x)
        return self.wq(h), self.wk(h), self.wv(h)

    def attend(self, q, k, v, rope):
        B, S, _ = q.shape
        q = q.view(B, S, self.heads, self.hd)
        k, v = k.view(B, S, self.kv_heads, self.hd), v.view(B, S, self.kv_heads, self.hd)
        if self.q_norm is not None:
            q, k = self.q_norm(q), self.k_norm(k)
        cos, sin = rope

        def rot(t):  # rotate pairs (even, odd) of the head dimension
            t2 = t.float().reshape(*t.shape[:-1], self.hd // 2, 2)
            a, b = t2[..., 0], t2[..., 1]
            return torch.stack((a * cos - b * sin, a * sin + b * cos), dim=-1).reshape(t.shape).to(t.dtype)

        q, k = rot(q), rot(k)
        o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                           is_causal=True, enable_gqa=True)
        return o.transpose(1, 2).reshape(B, S, self.dim)

    def forward(self, x, rope, norm):
        return self.wo(self.attend(*self.qkv(x, norm), rope))


class _Block(nn.Module):
    def __init__(self, dim, heads, kv_heads, ffn, eps, qk_norm=False):
        super().__init__()
        self.attention = _Attention(dim, heads, kv_heads, eps if qk_norm else None)
        self.feed_forward = FeedForward.Config(hidden_dim=ffn).build(dim=dim)
        self.attention_norm = nn.RMSNorm(dim, eps=eps)
        self.ffn_norm = nn.RMSNorm(dim, eps=eps)

    def ffn(self, h):
        ff = self.feed_forward
        w = (ff.w1.weight, ff.w2.weight, ff.w3.weight)
        if norm_fusable(h, self.ffn_norm.weight, w[0], w[2], for_feed_forward=True) and feed_forward_fusable(h, *w):
            return mx_norm_feed_forward(h, self.ffn_norm.weight, self.ffn_norm.eps, *w)
        return ff(self.ffn_norm(h))

    def forward(self, x, rope):
        h = x + self.attention(x, rope, self.attention_norm)
        return h + self.ffn(h)


def _rope(seq, hd, theta, device):
    pos = torch.arange(seq, device=device, dtype=torch.float32)
    freqs = 1.0 / (theta ** (torch.arange(0, hd, 2, device=device, dtype=torch.float32) / hd))
    ang = torch.outer(pos, freqs)[None, :, None, :]
    return ang.cos(), ang.sin()


class _OracleLinear(nn.Module):
    """y = emulated-MX x W^T computed by the CPU oracle from the raw bf16 values (forward only)."""

    def __init__(self, weight):
        super().__init__()
        self.weight = weight
        self.bias = None
        self.wq = co.cast_dim0(bits_of(weight), mo.RCEIL)

    def forward(self, x):
        x2 = x.reshape(-1, x.shape[-1])
        y = _oracle_matmul(*co.cast_dim0(bits_of(x2), mo.RCEIL), *self.wq)
        return bf16_from_bits(y, x.device).view(*x.shape[:-1], -1)


@pytest.mark.parametrize("norms_in_casts", [False, True])
def test_llama3_8b_block_at_seq_8192(device, norms_in_casts):
    """The whole block, forward + backward, at batch 1 x seq 8192 with random token ids from a
    vocabulary of 128 256 (the embedding row of each id is the block's input), against the same
    block with its seven linears replaced by the oracle's, on the first 256 tokens.

    Stage by stage on identical inputs: the three projections behind the attention norm, the output
    projection, and the feed-forward half, each as the block runs it at the full sequence.  Then
    the whole block.  A difference d in the input of a cast is re-rounded to e4m3 (step s of about
    2^-4 relative): a share d / s of the codes move by a whole step, so the difference behind the
    cast is about sqrt(d s), far more than d.  The feed-forward half holds one cast behind its two
    first GEMMs and the whole block four casts in a row, hence the wider bounds there; they are
    what the emulated recipe does to any two implementations that differ in summation order."""
    dim, heads, kv_heads, ffn, seq, vocab, head = 4096, 32, 8, 14336, 8192, 128256, 256
    torch.manual_seed(5)
    blk = _Block(dim, heads, kv_heads, ffn, 1e-5)
    _convert(blk, ["attention", "feed_forward"], fuse_rmsnorm_cast=norms_in_casts)
    blk.to(device).to(torch.bfloat16)
    with torch.no_grad():
        for m in blk.modules():
            if isinstance(m, nn.Linear):
                m.weight.normal_(0.0, 0.02)
    assert sum(isinstance(p, MXFP8TrainingWeight) for p in blk.parameters()) == 7
    att, ff = blk.attention, blk.feed_forward
    probe = torch.zeros(1, 32, dim, device=device, dtype=torch.bfloat16)
    assert norm_fusable(probe, blk.attention_norm.weight, att.wq.weight, att.wk.weight, att.wv.weight) == norms_in_casts
    assert norm_fusable(probe, blk.ffn_norm.weight, ff.w1.weight, ff.w3.weight) == norms_in_casts
    emb = nn.Embedding(vocab, dim, device=device, dtype=torch.bfloat16)
    tokens = torch.randint(0, vocab, (1, seq), device=device)
    x = emb(tokens).detach().requires_grad_(True)
    rope = _rope(seq, dim // heads, 500000.0, device)
    y = blk(x, rope)
    dy = torch.randn_like(y) * 1e-3
    y.backward(dy)
    assert torch.isfinite(y).all() and torch.isfinite(x.grad).all()
    for n, p in blk.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad).all() and float(p.grad.abs().max()) > 0, n

    # the backward as a whole: every gradient against the same block in plain bf16 (torch's linears
    # and autograd) on the same input and output gradient.  The two differ by the MXFP8 rounding of
    # every GEMM operand (about 3 % per operand, partly averaged out over the contraction), so a
    # wiring mistake (a missing term, a transposed operand, a wrong cast direction) is an order of
    # magnitude outside the bound
    plain = _Block(dim, heads, kv_heads, ffn, 1e-5).to(device).to(torch.bfloat16)
    plain.load_state_dict({k: v.detach().clone() for k, v in blk.state_dict().items()})
    xb = x.detach().clone().requires_grad_(True)
    plain(xb, rope).backward(dy)
    g_errs = {"x": rel_l2(x.grad.float().cpu().numpy(), xb.grad.float().cpu().numpy())}
    plain_grads = dict(plain.named_parameters())
    for n, p in blk.named_parameters():
        g_errs[n] = rel_l2(p.grad.float().cpu().numpy(), plain_grads[n].grad.float().cpu().numpy())
    print(f"rel-L2 of the gradients against the bf16 block: {g_errs}", flush=True)
    assert max(g_errs.values()) <= 0.2, g_errs  # observed: 0.07 (x, feed-forward weights) to 0.13 (attention weights)
    del plain, plain_grads, xb

    ref = _Block(dim, heads, kv_heads, ffn, 1e-5).to(device).to(torch.bfloat16)
    ref.load_state_dict(blk.state_dict())
    for parent, names in ((ref.attention, ("wq", "wk", "wv", "wo")), (ref.feed_forward, ("w1", "w2", "w3"))):
        for nme in names:
            setattr(parent, nme, _OracleLinear(getattr(parent, nme).weight.detach()))
    rope_head = (rope[0][:, :head], rope[1][:, :head])

    def err(got, want):
        return rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy())

    errs = {}
    with torch.no_grad():
        xd = x.detach()
        # wq / wk / wv behind the attention norm (inside the cast when norms_in_casts)
        for name, got, want in zip(("wq", "wk", "wv"), blk.attention.qkv(xd, blk.attention_norm),
                                   ref.attention.qkv(xd[:, :head], ref.attention_norm)):
            errs[name] = err(got[:, :head], want)
            assert errs[name] <= (2 * TOL if norms_in_casts else TOL), (name, errs)
        # wo on the attention output the block itself produced
        o = blk.attention.attend(*blk.attention.qkv(xd, blk.attention_norm), rope)
        errs["wo"] = err(blk.attention.wo(o)[:, :head], ref.attention.wo(o[:, :head]))
        assert errs["wo"] <= TOL, errs
        # the feed-forward half (norm, w1, w3, gate, w2) on the block's own residual stream
        h = xd + blk.attention.wo(o)
        errs["ffn"] = err(blk.ffn(h)[:, :head], ref.ffn(h[:, :head]))
        assert errs["ffn"] <= 6e-3, errs
        # the whole block
        want = ref(xd[:, :head], rope_head)
        errs["block"] = err(y.detach()[:, :head], want)
        # and without the residual stream, which carries most of the output's norm
        errs["block_minus_input"] = err(y.detach()[:, :head] - xd[:, :head], want - xd[:, :head])
        print(f"rel-L2 against the block built from oracle linears: {errs}", flush=True)
        assert errs["block"] <= 6e-2 and errs["block_minus_input"] <= 7e-2, errs  # observed 0.031 / 0.034


# ---- the policy step -------------------------------------------------------------------------
QWEN3_1P7B_LINEARS = {  # name: (in, out) at dim 2048, 16 heads / 8 KV heads of 128, FFN 6144
    "wq_wo": (2048, 2048), "wk_wv": (2048, 1024), "w1_w3": (2048, 6144), "w2": (6144, 2048)}
POLICY_TOKENS = 147456  # 128 sequences, lengths uniform in [256, 2048], packed (mean 1152)


@pytest.mark.parametrize("name", list(QWEN3_1P7B_LINEARS))
def test_qwen3_1p7b_layer_linears_over_the_packed_policy_step(device, name):
    """Every linear shape of one layer at 147 456 tokens, all three passes: the kv projection
    (N = 1024), the 6144 -> 2048 down projection, and the weight gradients whose contraction over
    the tokens is split over the CUs."""
    K, N = QWEN3_1P7B_LINEARS[name]
    x, w, dy, dw = _one_linear_at_size(device, POLICY_TOKENS, K, N, seed=K + N)
    # the weight gradient over all tokens against the sum of the gradients over two halves
    T = POLICY_TOKENS
    halves = torch.zeros_like(dw, dtype=torch.float32)
    for r0 in (0, T // 2):
        a = ops.to_mx_dim1(dy[r0:r0 + T // 2].contiguous(), "rceil", ops.MX_SCALES_MFMA)
        b = ops.to_mx_dim1(x[r0:r0 + T // 2].contiguous(), "rceil", ops.MX_SCALES_MFMA)
        halves += ops.mx_gemm_nt(a, b).float()
    # each half is rounded to bf16 before the sum: two roundings of 2^-9 relative against one
    assert rel_l2(dw.float().cpu().numpy(), halves.cpu().numpy()) <= 3e-3


def test_qwen3_1p7b_weight_hand_over_of_all_28_layers(device):
    """The re-cast of every converted weight of the 28-layer model for the hand-over in MXFP8 form:
    196 weights, 1.4 G elements.  Sampled rows of every payload entry bit-exact against the
    oracle's cast of the same rows of the weight."""
    dim, kv, ffn, layers = 2048, 1024, 6144, 28

    class Layer(nn.Module):
        def __init__(self):
            super().__init__()
            mk = lambda i, o: Linear.Config().build(in_features=i, out_features=o)
            self.attention = nn.Module()
            self.attention.wq, self.attention.wo = mk(dim, dim), mk(dim, dim)
            self.attention.wk, self.attention.wv = mk(dim, kv), mk(dim, kv)
            self.feed_forward = FeedForward.Config(hidden_dim=ffn).build(dim=dim)

    model = nn.Module()
    with torch.device("meta"):
        model.layers = nn.ModuleList([Layer() for _ in range(layers)])
    _convert(model, ["attention", "feed_forward"])
    model.to_empty(device=device)
    model.to(torch.bfloat16)
    g = torch.Generator(device=device).manual_seed(9)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_(torch.randn(p.shape, generator=g, device=device, dtype=torch.float32) * 0.02)
    converted = {n: p for n, p in model.named_parameters() if isinstance(p, MXFP8TrainingWeight)}
    assert len(converted) == 7 * layers
    payload = export_mxfp8_state_dict(model)
    rng = np.random.default_rng(4)
    sent = 0
    for name, p in converted.items():
        entry = payload[name]
        rows, cols = p.shape
        assert entry["codes"].shape == (rows, cols) and entry["scales"].shape == (rows, cols // 32)
        sent += entry["codes"].numel() + entry["scales"].numel()
        pick = np.sort(rng.choice(rows, size=16, replace=False))
        idx = torch.from_numpy(pick).to(device)
        plain = p.detach().as_subclass(torch.Tensor)
        c, s = mo.cast_dim0(bits_of(plain[idx]), mo.RCEIL)
        assert np.array_equal(entry["codes"][idx].cpu().numpy(), c), name
        assert np.array_equal(entry["scales"][idx].cpu().numpy(), s), name
    elements = sum(p.numel() for p in converted.values())
    assert elements == layers * (2 * dim * dim + 2 * dim * kv + 3 * dim * ffn) and sent * 32 == elements * 33


def test_token_log_probs_at_the_real_vocabulary_over_many_rows(device):
    """Forward and backward of the token log-probabilities at vocabulary 151 936 over 66 048 rows:
    more than the 65 535 rows one backward launch takes, so the chunking is on the path.  Sampled
    rows against the float64 oracle; every row's gradient sums to ~0 over the vocabulary times
    its upstream gradient (softmax gradients do), checked through a column sum."""
    from torchtitan_amd.rl.loss import token_log_probs

    rows, vocab = 66048, 151936
    torch.manual_seed(12)
    logits = torch.empty(rows, vocab, device=device, dtype=torch.bfloat16)
    for r0 in range(0, rows, 8192):  # filled in pieces: no float32 copy of the whole matrix
        logits[r0:r0 + 8192] = (torch.randn(min(8192, rows - r0), vocab, device=device) * 2.0).to(torch.bfloat16)
    logits.requires_grad_(True)
    target = torch.randint(0, vocab, (rows,), device=device)
    lp = token_log_probs(logits, target)
    g = torch.randn(rows, device=device)
    lp.backward(g)
    grad = logits.grad
    pick = np.array([0, 1, 4095, 32767, 65534, 65535, 65536, 66047])
    idx = torch.from_numpy(pick).to(device)
    lb = bits_of(logits.detach()[idx])
    tg = target[idx].cpu().numpy()
    want_lp, _ = mo.token_log_probs(lb, tg)
    assert np.allclose(lp.detach()[idx].cpu().numpy(), want_lp, rtol=0, atol=1e-5)
    want_g = mo.token_log_probs_grad(lb, tg, g[idx].cpu().numpy().astype(np.float64))
    got_g = grad[idx].float().cpu().numpy()
    # one bf16 step
    assert np.all(np.abs(got_g - want_g) <= np.maximum(np.abs(want_g) * 2.0 ** -7, 1e-30))
    # rows behind the first launch's 65 535 are written too, and no row is left at its initial value
    sums = torch.cat([grad[r0:r0 + 8192].float().sum(dim=1) for r0 in range(0, rows, 8192)])
    assert torch.isfinite(sums).all()
    mags = torch.cat([grad[r0:r0 + 8192].abs().amax(dim=1).float() for r0 in range(0, rows, 8192)])
    assert bool((mags[g != 0] > 0).all())
    # sum_v dlogits[r, v] = g[r] (1 - sum softmax) ~ 0 up to the bf16 rounding of 151 936 entries
    assert float((sums.abs() / g.abs().clamp_min(1e-3)).max()) < 0.05


def test_policy_step_composed_at_real_layer_shapes(device):
    """benchmark configs[4] composed, at the real layer shapes on two layers: 16 sequences (2 prompts
    x 8 samples) of uneven lengths uniform in [256, 2048] with random token ids below 151 936,
    each through embedding -> two Qwen3-1.7B-shaped layers (dim 2048, 16 heads / 8 KV heads of
    128 with q/k norms, FFN 6144, all seven linears MXFP8, the SwiGLU block fused) -> norm ->
    language-model head at the full vocabulary -> fused token log-probabilities, into
    `compute_policy_gradient_loss` with advantages = reward - group mean; backward; an optimizer
    step; the MXFP8 hand-over of the updated weights.

    Checked: the loss and its metrics against the float64 oracle on the model's own log-probs; one
    sequence's log-probs against the oracle's log-softmax of the same logits; on the first 256
    tokens of the longest sequence every stage of both layers against the same stage built from
    oracle linears on identical inputs (as for the Llama block above); every gradient finite and
    non-zero and the same from a second run; the payload of sampled weights bit-exact against the
    oracle's cast of the updated weight."""
    import math

    from torchtitan_amd.rl import compute_policy_gradient_loss, token_log_probs

    dim, heads, kv_heads, ffn, vocab, eps, head = 2048, 16, 8, 6144, 151936, 1e-6, 256

    class PolicyLM(nn.Module):
        def __init__(self):
            super().__init__()
            self.tok_embeddings = nn.Embedding(vocab, dim)
            self.layers = nn.ModuleList([_Block(dim, heads, kv_heads, ffn, eps, qk_norm=True) for _ in range(2)])
            self.norm = nn.RMSNorm(dim, eps=eps)
            self.output = Linear.Config().build(in_features=dim, out_features=vocab)
            self.hidden = None  # inputs of the layers of the last forward, for the stage checks

        def forward(self, tokens, attention_masks=None):
            h = self.tok_embeddings(tokens)
            S = h.shape[1]
            pad = -S % 32  # the MXFP8 linears take multiples of 32 tokens; causal: real positions do not see the padding
            if pad:
                h = torch.cat((h, h.new_zeros((1, pad, dim))), dim=1)
            rope = _rope(S + pad, dim // heads, 1000000.0, h.device)
            self.hidden = []
            for layer in self.layers:
                self.hidden.append(h.detach())
                h = layer(h, rope)
            return self.output(self.norm(h[:, :S]))

    torch.manual_seed(15)
    model = PolicyLM()
    box = ModelConvertersContainer.Config(
        converters=[MXFP8Converter.Config(fqns=["attention", "feed_forward"], recipe_name="mxfp8_rceil")]
    ).build(parallel_dims=None, model_compile_enabled=False)
    box.convert(model)
    model.to(device).to(torch.bfloat16)
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, nn.Linear):
                m.weight.normal_(0.0, 0.02)
        model.tok_embeddings.weight.normal_(0.0, 1.0)
    converted = {n: p for n, p in model.named_parameters() if isinstance(p, MXFP8TrainingWeight)}
    assert len(converted) == 14 and "output.weight" not in converted

    rng = np.random.default_rng(21)
    total_len = rng.integers(256, 2049, 16)
    total_len[3] = 2048  # one sequence at the upper end, one that needs padding to 32
    total_len[5] = 333
    prompts, gens = [], []
    for i, L in enumerate(total_len):
        p_len = int(rng.integers(16, 65)) if i % 8 else 32  # samples of a group share a prompt length
        ids = rng.integers(0, vocab, int(L)).tolist()
        prompts.append(ids[:p_len])
        gens.append(ids[p_len:])
    rewards = torch.tensor(rng.standard_normal(16), dtype=torch.float32)
    adv = (rewards.view(2, 8) - rewards.view(2, 8).mean(dim=1, keepdim=True)).view(-1)

    with torch.no_grad():  # the reference policy's log-probs: the same model, shifted a little
        ref = []
        for i, (p, g) in enumerate(zip(prompts, gens)):
            logits = model(torch.tensor([p + g], device=device))[0, len(p) - 1:len(p) - 1 + len(g)]
            tgt = torch.tensor(g, device=device)
            lp = token_log_probs(logits, tgt)
            ref.append(lp + 0.05 * torch.randn(lp.shape, device=device, generator=None))
            if i == 5:  # one sequence against the oracle's float64 log-softmax of the same logits (sampled rows)
                rows = np.sort(rng.choice(len(g), size=24, replace=False))
                want, _ = mo.token_log_probs(bits_of(logits[torch.from_numpy(rows).to(device)]), np.array(g)[rows])
                assert np.abs(lp[torch.from_numpy(rows).to(device)].cpu().numpy() - want).max() <= 1e-5

    def step():
        for p in model.parameters():
            p.grad = None
        total, metrics, lps = compute_policy_gradient_loss(model, gens, prompts, adv, ref)
        total.backward()
        return total, metrics, lps

    total, metrics, lps = step()
    o_total, o_m = mo.policy_gradient_loss([l.detach().cpu().numpy() for l in lps], [r.cpu().numpy() for r in ref],
                                           adv.numpy())
    assert math.isclose(total.item(), o_total, rel_tol=1e-4, abs_tol=1e-5)
    for k in ("pg_loss", "entropy", "kl_div", "ratio_mean"):
        assert math.isclose(metrics[k], o_m[k], rel_tol=1e-3, abs_tol=1e-5), k
    grads = {n: p.grad.clone() for n, p in model.named_parameters()}
    for n, gr in grads.items():
        assert torch.isfinite(gr).all() and float(gr.abs().max()) > 0, n
    total2, _, _ = step()
    assert total2.item() == total.item()
    for n, p in model.named_parameters():
        assert torch.equal(p.grad, grads[n]), n

    # stage by stage on the first 256 tokens of the longest sequence, inputs as the model produced them
    with torch.no_grad():
        i = 3
        model(torch.tensor([prompts[i] + gens[i]], device=device))
        rope = _rope(2048, dim // heads, 1000000.0, device)
        rope_head = (rope[0][:, :head], rope[1][:, :head])
        err = lambda got, want: rel_l2(got.float().cpu().numpy(), want.float().cpu().numpy())
        for li, (blk, xd) in enumerate(zip(model.layers, model.hidden)):
            ref_blk = _Block(dim, heads, kv_heads, ffn, eps, qk_norm=True).to(device).to(torch.bfloat16)
            ref_blk.load_state_dict(blk.state_dict())
            for parent, names in ((ref_blk.attention, ("wq", "wk", "wv", "wo")), (ref_blk.feed_forward, ("w1", "w2", "w3"))):
                for nme in names:
                    setattr(parent, nme, _OracleLinear(getattr(parent, nme).weight.detach()))
            errs = {}
            for name, got, want in zip(("wq", "wk", "wv"), blk.attention.qkv(xd, blk.attention_norm),
                                       ref_blk.attention.qkv(xd[:, :head], ref_blk.attention_norm)):
                errs[name] = err(got[:, :head], want)
                assert errs[name] <= TOL, (li, name, errs)
            o = blk.attention.attend(*blk.attention.qkv(xd, blk.attention_norm), rope)
            errs["wo"] = err(blk.attention.wo(o)[:, :head], ref_blk.attention.wo(o[:, :head]))
            assert errs["wo"] <= TOL, (li, errs)
            h = xd + blk.attention.wo(o)
            errs["ffn"] = err(blk.ffn(h)[:, :head], ref_blk.ffn(h[:, :head]))
            assert errs["ffn"] <= 6e-3, (li, errs)
            # the layer without its residual stream (which would hide everything else)
            errs["layer_minus_input"] = err(blk(xd, rope)[:, :head] - xd[:, :head], ref_blk(xd[:, :head], rope_head) - xd[:, :head])
            print(f"layer {li}: rel-L2 against the stages built from oracle linears: {errs}", flush=True)
            assert errs["layer_minus_input"] <= 3e-2, (li, errs)
            del ref_blk

    # optimizer step, then the hand-over of the updated weights
    with torch.no_grad():
        for p in model.parameters():
            p.add_(p.grad, alpha=-1.0)
    box.post_optimizer_hook(model)
    payload = export_mxfp8_state_dict(model)
    for name in ("layers.0.attention.wk.weight", "layers.1.feed_forward.w2.weight", "layers.1.feed_forward.w1.weight"):
        p = converted[name]
        plain = p.detach().as_subclass(torch.Tensor)
        pick = torch.from_numpy(np.sort(rng.choice(p.shape[0], size=16, replace=False))).to(device)
        c, s_ = mo.cast_dim0(bits_of(plain[pick]), mo.RCEIL)
        assert np.array_equal(payload[name]["codes"][pick].cpu().numpy(), c), name
        assert np.array_equal(payload[name]["scales"][pick].cpu().numpy(), s_), name
    assert set(payload) >= set(converted)
