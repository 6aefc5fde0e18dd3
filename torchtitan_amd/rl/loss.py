"""GRPO / PPO policy-gradient loss with per-token KL, and the per-token log-probabilities under
it (torchtitan/experiments/rl/unified/actors/utils.py:11-147).

Same functions, arguments, return values and formulas as the reference.  The one heavy step,
log-softmax over the vocabulary in float32 followed by a gather of the generated tokens, runs
as one HIP kernel over the bf16 logits (and one more in backward) whenever the logits are a
bf16 GPU tensor; otherwise the same torch ops as the reference run.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from .. import ops


class _TokenLogProbs(torch.autograd.Function):
    """log_softmax(logits.float(), -1).gather(1, target[:, None]).squeeze(-1) for bf16 logits."""

    @staticmethod
    def forward(ctx, logits, target):
        lp, lse = ops.token_logprob_fwd(logits, target)
        ctx.save_for_backward(logits, target, lse)
        return lp

    @staticmethod
    def backward(ctx, grad):
        logits, target, lse = ctx.saved_tensors
        return ops.token_logprob_bwd(logits, target, lse, grad), None


def token_log_probs(logits: torch.Tensor, target: torch.Tensor) -> torch.Tensor:
    """float32 log-probability of target[r] under softmax(logits[r]); logits [rows, vocab]."""
    if logits.is_cuda and logits.dtype == torch.bfloat16 and logits.dim() == 2:
        return _TokenLogProbs.apply(logits, target)
    log_probs = F.log_softmax(logits.to(torch.float32), dim=-1)
    return log_probs.gather(1, target.unsqueeze(-1)).squeeze(-1)


def compute_token_log_probs(model: torch.nn.Module, prompt_token_ids: list[int],
                            gen_token_ids: list[int], device: torch.device) -> torch.Tensor:
    """Per-token log-probabilities of the generated tokens under `model` (one forward over
    prompt + completion; position i predicts token i + 1)."""
    full = torch.tensor(prompt_token_ids + gen_token_ids, dtype=torch.long, device=device).unsqueeze(0)
    logits = model(full, attention_masks=None)
    start = len(prompt_token_ids) - 1
    stop = start + len(gen_token_ids)
    return token_log_probs(logits[0, start:stop, :], full[0, start + 1:stop + 1])


def compute_policy_gradient_loss(model: torch.nn.Module, vllm_token_ids: list[list[int]],
                                 prompt_token_ids: list[list[int]], advantages: torch.Tensor,
                                 ref_token_log_probs: list[torch.Tensor], kl_coef: float = 0.1,
                                 ppo_clip_eps: float = 0.2, entropy_coef: float = 0.01):
    """(total loss, metrics dict, per-sample policy log-probs).

    Per sample: mean over its tokens of log(pi / pi_ref) -> ratio; clipped PPO objective on that
    ratio; KL by the k3 estimator ratio - 1 - log ratio per token, averaged per sample, then over
    samples; entropy bonus from the mean log-probability of all tokens."""
    device = next(model.parameters()).device
    advantages = advantages.to(device)
    batch_lps = [compute_token_log_probs(model, p, g, device) for p, g in zip(prompt_token_ids, vllm_token_ids)]
    mean_log_ratio, mean_kl = [], []
    for lps, ref in zip(batch_lps, ref_token_log_probs):
        log_ratio = lps - ref.detach()
        mean_log_ratio.append(log_ratio.mean())
        mean_kl.append((torch.exp(log_ratio) - 1 - log_ratio).mean())
    mean_log_ratio, mean_kl = torch.stack(mean_log_ratio), torch.stack(mean_kl)
    ratio = torch.exp(mean_log_ratio)
    clipped_ratio = torch.clamp(ratio, 1 - ppo_clip_eps, 1 + ppo_clip_eps)
    pg_loss = -torch.min(ratio * advantages, clipped_ratio * advantages).mean()
    entropy = -torch.cat(batch_lps).mean()
    kl_div = mean_kl.mean()
    total = pg_loss + (-entropy_coef * entropy) + kl_coef * kl_div
    metrics = {
        "pg_loss": pg_loss.item(),
        "entropy": entropy.item(),
        "kl_div": kl_div.item(),
        "ratio_mean": ratio.mean().item(),
        "ratio_clipped_frac": (torch.abs(ratio - clipped_ratio) > 1e-6).float().mean().item(),
    }
    return total, metrics, batch_lps
