"""GPU parity of the fused token log-probability kernels and of the loss around them."""
import math

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import mx_oracle as mo
from tests.helpers import bf16_from_bits, bits_of, rel_l2
from torchtitan_amd import ops
from torchtitan_amd.rl import compute_policy_gradient_loss, token_log_probs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,vocab", [(5, 64), (33, 1003), (64, 50257), (48, 151936)])
def test_token_logprob_kernels_vs_oracle(device, rows, vocab):
    """float32 log-sum-exp over bf16 logits: log-probs within 1e-5 of the float64 oracle; the
    gradient within one bf16 step of the oracle's, elementwise."""
    rng = np.random.default_rng(rows + vocab)
    bits = mo.f32_to_bf16_bits((rng.standard_normal((rows, vocab)) * 4).astype(np.float32))
    bits[0, : min(vocab, 40)] = mo.f32_to_bf16_bits(np.float32(60.0))  # a peaked row
    target = rng.integers(0, vocab, rows)
    target[0] = 3
    logits = bf16_from_bits(bits, device)
    if vocab % 8:
        assert logits.stride(0) % 8
    t = torch.from_numpy(target).to(device)
    lp, lse = ops.token_logprob_fwd(logits, t)
    lp_o, lse_o = mo.token_log_probs(bits, target)
    assert np.abs(lp.cpu().numpy() - lp_o).max() <= 1e-5
    assert np.abs(lse.cpu().numpy() - lse_o).max() <= 1e-5
    g = rng.standard_normal(rows).astype(np.float32)
    d = ops.token_logprob_bwd(logits, t, lse, torch.from_numpy(g).to(device))
    d_o = mo.token_log_probs_grad(bits, target, g.astype(np.float64))
    got = mo.bf16_bits_to_f32(bits_of(d)).astype(np.float64)
    assert (np.abs(got - d_o) <= np.abs(d_o) * 2.0 ** -7 + 1e-12).all()
    assert rel_l2(got, d_o) <= 3e-3


def test_token_log_probs_autograd_matches_torch_ops(device):
    torch.manual_seed(1)
    x = (torch.randn(70, 4099, device=device) * 3).to(torch.bfloat16)
    tgt = torch.randint(0, 4099, (70,), device=device)
    a, b = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    w = torch.randn(70, device=device)
    la = token_log_probs(a, tgt)
    lb = F.log_softmax(b.to(torch.float32), dim=-1).gather(1, tgt[:, None]).squeeze(-1)
    assert torch.allclose(la, lb, atol=1e-5)
    (la * w).sum().backward()
    (lb * w).sum().backward()
    assert rel_l2(a.grad.float().cpu().numpy(), b.grad.float().cpu().numpy()) <= 3e-3
    assert type(la.grad_fn).__name__ == "_TokenLogProbsBackward"


class _ToyLM(nn.Module):
    def __init__(self, vocab=1000, dim=64):
        super().__init__()
        self.emb = nn.Embedding(vocab, dim)
        self.out = nn.Linear(dim, vocab, bias=False)

    def forward(self, tokens, attention_masks=None):
        h = self.emb(tokens)
        return self.out(h + h.cumsum(dim=1) * 0.1)


def test_policy_gradient_loss_fused_vs_oracle(device):
    """The whole loss on a small bf16 model: per-token log-probs from the fused kernel, loss and
    metrics against the float64 oracle fed with the oracle's own log-probs of the same logits."""
    torch.manual_seed(2)
    model = _ToyLM().to(device).to(torch.bfloat16)
    rng = np.random.default_rng(4)
    prompts = [rng.integers(0, 1000, n).tolist() for n in (5, 9, 3, 7)]
    gens = [rng.integers(0, 1000, n).tolist() for n in (12, 30, 8, 17)]
    adv = torch.tensor([0.5, -0.2, 1.5, -1.0])
    lps_o, ref = [], []
    for p, g in zip(prompts, gens):
        full = torch.tensor([p + g], device=device)
        with torch.no_grad():
            logits = model(full)[0, len(p) - 1:len(p) - 1 + len(g)]
        lp, _ = mo.token_log_probs(bits_of(logits), np.array(g))
        lps_o.append(lp)
        ref.append(torch.from_numpy(lp + 0.1 * rng.standard_normal(len(g))).float().to(device))
    total, metrics, lps = compute_policy_gradient_loss(model, gens, prompts, adv, ref)
    for got, want in zip(lps, lps_o):
        assert np.abs(got.detach().cpu().numpy() - want).max() <= 1e-5
        assert type(got.grad_fn).__name__ == "_TokenLogProbsBackward"
    o_total, o_m = mo.policy_gradient_loss(lps_o, [r.cpu().numpy() for r in ref], adv.numpy())
    assert math.isclose(total.item(), o_total, rel_tol=1e-4, abs_tol=1e-5)
    for k, v in o_m.items():
        assert math.isclose(metrics[k], v, rel_tol=1e-4, abs_tol=1e-5), k
    total.backward()
    assert torch.isfinite(model.out.weight.grad).all() and model.out.weight.grad.abs().sum() > 0


def test_policy_step_on_a_small_converted_model_then_weight_hand_over(device):
    """benchmark configs[4] in small: a dense decoder-only model with MXFP8 linears, packed
    prompts / completions of different lengths, the policy-gradient loss on fused log-probs,
    backward, an optimizer step, then the re-cast of all converted weights for the hand-over."""
    from tests.test_converter_gpu import _MiniDecoderBlock
    from torchtitan_amd import ops
    from torchtitan_amd.modules import Linear
    from torchtitan_amd.mx_tensor import MXFP8TrainingWeight
    from torchtitan_amd.protocols import ModelConvertersContainer
    from torchtitan_amd.quantization.mx import MXFP8Converter, export_mxfp8_state_dict, load_mxfp8_state_dict

    vocab, dim = 512, 128

    class TinyLM(nn.Module):
        def __init__(self):
            super().__init__()
            self.tok_embeddings = nn.Embedding(vocab, dim)
            self.layers = nn.ModuleList([_MiniDecoderBlock(dim, 4, 2, 256) for _ in range(2)])
            self.norm = nn.RMSNorm(dim, eps=1e-5)
            self.output = Linear.Config().build(in_features=dim, out_features=vocab)

        def forward(self, tokens, attention_masks=None):
            h = self.tok_embeddings(tokens)
            # the MXFP8 linears want a multiple of 32 tokens: pad the sequence on the right
            # (causal attention: the real positions do not see the padding)
            S = h.shape[1]
            pad = -S % 32
            if pad:
                h = torch.cat((h, h.new_zeros((1, pad, dim))), dim=1)
            for layer in self.layers:
                h = layer(h)
            return self.output(self.norm(h[:, :S]))

    torch.manual_seed(3)
    model = TinyLM().to(device).to(torch.bfloat16)
    box = ModelConvertersContainer.Config(
        converters=[MXFP8Converter.Config(fqns=["attention", "feed_forward"], cache_weight_casts=True)]
    ).build(parallel_dims=None, model_compile_enabled=False)
    box.convert(model)
    assert sum(isinstance(p, MXFP8TrainingWeight) for p in model.parameters()) == 14
    rng = np.random.default_rng(6)
    prompts = [rng.integers(0, vocab, n).tolist() for n in (7, 20, 12)]
    gens = [rng.integers(0, vocab, n).tolist() for n in (25, 9, 40)]
    adv = torch.tensor([1.0, -0.5, 0.25])
    with torch.no_grad():
        ref = [token_log_probs(model(torch.tensor([p + g], device=device))[0, len(p) - 1:len(p) - 1 + len(g)],
                               torch.tensor(g, device=device)) + 0.05 for p, g in zip(prompts, gens)]
    total, metrics, lps = compute_policy_gradient_loss(model, gens, prompts, adv, ref)
    o_total, o_m = mo.policy_gradient_loss([l.detach().cpu().numpy() for l in lps], [r.cpu().numpy() for r in ref],
                                           adv.numpy())
    assert math.isclose(total.item(), o_total, rel_tol=1e-4, abs_tol=1e-5)
    assert math.isclose(metrics["kl_div"], o_m["kl_div"], rel_tol=1e-3, abs_tol=1e-6)
    total.backward()
    before = {n: p.detach().clone() for n, p in model.named_parameters()}
    with torch.no_grad():
        for p in model.parameters():
            assert p.grad is not None and torch.isfinite(p.grad).all()
            p.add_(p.grad, alpha=-0.5)
    box.post_optimizer_hook(model)
    payload = export_mxfp8_state_dict(model)
    restored = load_mxfp8_state_dict(payload)
    n_mx = 0
    for name, p in model.named_parameters():
        plain = p.detach().as_subclass(torch.Tensor)
        if isinstance(p, MXFP8TrainingWeight):
            n_mx += 1
            assert not torch.equal(plain, before[name])                 # the step moved it
            q = ops.to_mx_dim0(plain, "rceil", ops.MX_SCALES_ROWMAJOR)   # cast of the NEW weight
            assert torch.equal(payload[name]["codes"], q.codes) and torch.equal(payload[name]["scales"], q.scales)
            assert torch.equal(restored[name], ops.mx_dequant(q))
        else:
            assert torch.equal(restored[name], plain)
    assert n_mx == 14
