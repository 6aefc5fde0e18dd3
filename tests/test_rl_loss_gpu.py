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
