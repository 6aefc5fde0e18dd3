"""CPU: the policy-gradient loss mirror and its oracle (actors/utils.py:11-147) against torch's
own ops, closed forms and a hand example."""
import math

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import mx_oracle as mo
from torchtitan_amd.rl import compute_policy_gradient_loss, compute_token_log_probs


class _ToyLM(nn.Module):
    def __init__(self, vocab=97, dim=16):
        super().__init__()
        self.emb = nn.Embedding(vocab, dim)
        self.out = nn.Linear(dim, vocab, bias=False)

    def forward(self, tokens, attention_masks=None):
        h = self.emb(tokens)
        return self.out(h + h.cumsum(dim=1) * 0.1)


def test_oracle_token_log_probs_vs_torch_log_softmax_and_autograd():
    rng = np.random.default_rng(0)
    bits = mo.f32_to_bf16_bits((rng.standard_normal((40, 1003)) * 3).astype(np.float32))
    target = rng.integers(0, 1003, 40)
    lp, lse = mo.token_log_probs(bits, target)
    x = torch.from_numpy(mo.bf16_bits_to_f32(bits)).requires_grad_(True)
    ref = F.log_softmax(x, dim=-1).gather(1, torch.from_numpy(target)[:, None]).squeeze(-1)
    assert np.allclose(lp, ref.detach().numpy(), atol=2e-6)
    assert np.allclose(lse, torch.logsumexp(x, -1).detach().numpy(), atol=2e-6)
    g = rng.standard_normal(40)
    ref.backward(torch.from_numpy(g).float())
    assert np.allclose(mo.token_log_probs_grad(bits, target, g), x.grad.numpy(), atol=2e-6)


def test_oracle_loss_closed_forms_and_hand_example():
    lps = [np.array([-1.0, -2.0, -0.5]), np.array([-3.0, -0.25])]
    adv = np.array([0.7, -1.3])
    total, m = mo.policy_gradient_loss(lps, lps, adv)        # policy == reference
    assert m["kl_div"] == 0 and m["ratio_mean"] == 1 and m["ratio_clipped_frac"] == 0
    assert math.isclose(m["pg_loss"], -adv.mean()) and math.isclose(m["entropy"], 6.75 / 5)
    assert math.isclose(total, -adv.mean() - 0.01 * 6.75 / 5)
    # one sample, one token, log-ratio ln 2: ratio 2 clipped to 1.2 for a positive advantage
    total, m = mo.policy_gradient_loss([np.array([math.log(0.5)])], [np.array([math.log(0.25)])], np.array([1.0]))
    assert math.isclose(m["pg_loss"], -1.2) and math.isclose(m["kl_div"], 2 - 1 - math.log(2))
    assert m["ratio_clipped_frac"] == 1.0
    assert math.isclose(total, -1.2 - 0.01 * math.log(2) + 0.1 * (1 - math.log(2)))
    # negative advantage: min() keeps the unclipped term
    _, m = mo.policy_gradient_loss([np.array([math.log(0.5)])], [np.array([math.log(0.25)])], np.array([-1.0]))
    assert math.isclose(m["pg_loss"], 2.0)


def test_mirror_on_cpu_matches_oracle_and_reference_formulas():
    torch.manual_seed(0)
    model = _ToyLM()
    prompts = [[1, 5, 9], [2, 2], [7, 8, 9, 10]]
    gens = [[4, 4, 60], [11, 12, 13, 14, 15], [96]]
    with torch.no_grad():
        ref = [compute_token_log_probs(model, p, g, torch.device("cpu")) + 0.05 * (i - 1)
               for i, (p, g) in enumerate(zip(prompts, gens))]
    adv = torch.tensor([0.5, -0.2, 1.5])
    total, metrics, lps = compute_policy_gradient_loss(model, gens, prompts, adv, ref)
    # token log-probs: position i predicts token i + 1
    full = torch.tensor([prompts[0] + gens[0]])
    lp_all = F.log_softmax(model(full)[:, :-1].float(), -1)
    want = lp_all[0, 2:5].gather(1, torch.tensor(gens[0])[:, None]).squeeze(-1)
    assert torch.allclose(lps[0], want, atol=1e-6)
    o_total, o_m = mo.policy_gradient_loss([l.detach().numpy() for l in lps], [r.numpy() for r in ref], adv.numpy())
    assert math.isclose(total.item(), o_total, rel_tol=1e-5, abs_tol=1e-6)
    for k, v in o_m.items():
        assert math.isclose(metrics[k], v, rel_tol=1e-5, abs_tol=1e-6), k
    total.backward()
    assert model.out.weight.grad.abs().sum() > 0
