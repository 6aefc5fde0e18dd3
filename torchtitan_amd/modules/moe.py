"""Grouped experts and the token-group padding around ``torch._grouped_mm``.

Counterparts of ``GroupedExperts`` / ``_run_experts_grouped_mm`` / ``_run_experts_for_loop``
(torchtitan/models/common/moe/moe.py:24-134) and of ``_permute`` / ``_unpermute`` /
``indices_padding_wrapper`` / ``generate_permute_indices``
(torchtitan/models/common/moe/utils.py:17-120, moe/kernels.py:145-218).  The index fill runs in
the HIP library; ``use_cpu=True`` selects the host loop the reference keeps for comparison.
"""
from __future__ import annotations

from collections.abc import Callable
from typing import Literal

import torch
import torch.nn.functional as F
from torch import nn

from dataclasses import dataclass

from ..mx_blocks import (grouped_experts_align_themselves, grouped_feed_forward_fusable,
                         mx_grouped_feed_forward, mx_routed_experts)
from ..mx_tensor import grouped_mm
from ..protocols import Module
from .feed_forward import FeedForward
from .linear import Linear
from ..quantization import MXFP8_GROUP_ALIGNMENT_SIZE

TOKEN_GROUP_ALIGN_SIZE_M = 8
ValidTokenGroupAlignmentSize = Literal[8, 16, 32]


def _round_up(x: int, a: int) -> int:
    return -(-x // a) * a


def set_token_group_alignment_size_m(alignment_size: ValidTokenGroupAlignmentSize) -> None:
    """8 suffices for bf16, 16 for fp8, 32 for MXFP8 (wgrad contracts over tokens in blocks of 32)."""
    global TOKEN_GROUP_ALIGN_SIZE_M
    TOKEN_GROUP_ALIGN_SIZE_M = alignment_size


def get_mxfp8_pad_multiple() -> int | None:
    return MXFP8_GROUP_ALIGNMENT_SIZE if TOKEN_GROUP_ALIGN_SIZE_M == MXFP8_GROUP_ALIGNMENT_SIZE else None


def fill_indices_cpu(tokens_per_expert_group, start_index_values, write_offsets,
                     experts_per_rank: int, num_ranks: int, max_len: int) -> torch.Tensor:
    """Host loop with the semantics of the reference's CPU fill (moe/kernels.py:108-142)."""
    out = torch.full((max_len,), -1, dtype=torch.int64)
    for e in range(experts_per_rank):
        pos = int(write_offsets[e])
        for r in range(num_ranks):
            i = r * experts_per_rank + e
            n = int(tokens_per_expert_group[i])
            stop = min(pos + n, max_len)
            if n > 0 and pos < stop:
                first = int(start_index_values[i])
                out[pos:stop] = torch.arange(first, first + stop - pos, dtype=torch.int64)
            pos += n
    return out


def generate_permute_indices(tokens_per_expert_group: torch.Tensor, experts_per_rank: int,
                             num_ranks: int, max_len: int, alignment: int, use_cpu: bool = False):
    """(permuted_indices, m_sizes int32, m_offsets int32): expert-grouped, alignment-padded order."""
    if not use_cpu:
        if torch.compiler.is_compiling():  # the same launch as a graph node
            from .. import compiled

            return torch.ops.torchtitan_amd.group_offsets_pad(tokens_per_expert_group, experts_per_rank,
                                                              num_ranks, max_len, alignment)
        # product path: one HIP launch, no host round trip; raises on CPU tensors
        from .. import ops

        return ops.group_offsets_pad(tokens_per_expert_group, experts_per_rank, num_ranks, max_len, alignment)
    # explicit host reference, the counterpart of the reference's `use_cpu=True`
    t = tokens_per_expert_group.cpu()
    start = torch.cumsum(t, 0) - t
    per_expert = torch.clamp_min(t.view(num_ranks, -1).sum(0), alignment)
    m_sizes = ((per_expert + alignment - 1) // alignment * alignment).to(torch.int32)
    m_offsets = torch.cumsum(m_sizes, 0)
    perm = fill_indices_cpu(t, start, m_offsets - m_sizes, experts_per_rank, num_ranks, max_len)
    return perm, m_sizes, m_offsets.to(torch.int32)


def _permute(x, num_tokens_per_expert, ep_degree, num_local_experts):
    a = TOKEN_GROUP_ALIGN_SIZE_M
    max_len = _round_up(x.shape[0] + num_local_experts * a, a)
    with torch.no_grad():
        perm, m_sizes, _ = generate_permute_indices(num_tokens_per_expert, num_local_experts,
                                                    ep_degree, max_len, a)
    x = torch.vstack((x, x.new_zeros((x.shape[-1]))))  # row -1 of the source = zeros
    shape = x.shape
    return shape, x[perm, :], perm, m_sizes


def _unpermute(out, input_shape, permuted_indices):
    full = out.new_empty(input_shape)
    full[permuted_indices, :] = out
    return full[:-1]


def indices_padding_wrapper(func: Callable) -> Callable:
    """Pad every expert's token group to TOKEN_GROUP_ALIGN_SIZE_M before `func`, undo after."""

    def wrapper(w1, w2, w3, x, num_tokens_per_expert):
        n_local = w1.shape[0]
        ep_degree = num_tokens_per_expert.shape[0] // n_local
        shape, x, perm, num_tokens_per_expert = _permute(x, num_tokens_per_expert, ep_degree, n_local)
        out = func(w1, w2, w3, x, num_tokens_per_expert)
        return _unpermute(out, shape, perm)

    return wrapper


def _run_experts_for_loop(w1, w2, w3, x, num_tokens_per_expert):
    counts = num_tokens_per_expert.tolist()
    used = sum(counts)
    outs = []
    for e, xe in enumerate(torch.split(x[:used], counts, dim=0)):
        h = F.silu(xe @ w1[e].transpose(-2, -1)) * (xe @ w3[e].transpose(-2, -1))
        outs.append(h @ w2[e].transpose(-2, -1))
    out = torch.cat(outs, dim=0)
    return torch.vstack((out, out.new_zeros((x.shape[0] - used, out.shape[-1]))))


def _run_experts_grouped_mm(w1, w2, w3, x, num_tokens_per_expert):
    offsets = torch.cumsum(num_tokens_per_expert, dim=0, dtype=torch.int32)
    if grouped_feed_forward_fusable(x, w1, w2, w3):  # converted experts: one fused function
        return mx_grouped_feed_forward(x, w1, w2, w3, offsets).type_as(x)
    xb = x.bfloat16()
    # grouped_mm is torch._grouped_mm, spelled so that converted weights keep their MXFP8 path
    # inside a compiled graph as well
    h = F.silu(grouped_mm(xb, w1.bfloat16().transpose(-2, -1), offsets))
    h = h * grouped_mm(xb, w3.bfloat16().transpose(-2, -1), offsets)
    return grouped_mm(h, w2.bfloat16().transpose(-2, -1), offsets).type_as(x)


class GroupedExperts(Module):
    """E experts with 3-D parameters w1, w3: [E, hidden, dim] and w2: [E, dim, hidden]."""

    def __init__(self, *, dim: int, hidden_dim: int, num_experts: int, use_grouped_mm: bool):
        super().__init__()
        self.num_experts = num_experts
        self.w1 = nn.Parameter(torch.empty(num_experts, hidden_dim, dim))
        self.w2 = nn.Parameter(torch.empty(num_experts, dim, hidden_dim))
        self.w3 = nn.Parameter(torch.empty(num_experts, hidden_dim, dim))
        self.use_grouped_mm = use_grouped_mm

    def forward(self, x: torch.Tensor, num_tokens_per_expert: torch.Tensor) -> torch.Tensor:
        if self.use_grouped_mm:
            run = indices_padding_wrapper(_run_experts_grouped_mm)
            if num_tokens_per_expert.shape[0] == self.w1.shape[0] and (
                    (grouped_feed_forward_fusable(x, self.w1, self.w2, self.w3)
                     and self.w2.mx_config.pad_token_groups_for_grouped_mm)
                    or (torch.compiler.is_compiling()
                        and grouped_experts_align_themselves(self.w1, self.w2, self.w3))):
                # tokens already in expert order and the converted block aligns the groups itself
                run = _run_experts_grouped_mm
        else:
            run = _run_experts_for_loop
        return run(self.w1, self.w2, self.w3, x, num_tokens_per_expert)

    def init_weights(self, **kwargs) -> None:
        init_std = kwargs.get("init_std")
        assert init_std is not None
        nn.init.trunc_normal_(self.w1, mean=0.0, std=0.02)
        nn.init.trunc_normal_(self.w2, mean=0.0, std=init_std)
        nn.init.trunc_normal_(self.w3, mean=0.0, std=init_std)


class TokenChoiceTopKRouter(Module):
    """Token-choice routing: every token goes to its top_k experts by router score, optionally
    restricted to the best `num_limited_groups` of `num_expert_groups` expert groups
    (torchtitan/models/common/moe/moe.py:137-315).  Gate and scores run in float32."""

    def __init__(self, *, dim: int, num_experts: int, num_expert_groups: int | None,
                 num_limited_groups: int | None, top_k: int, score_func: Literal["softmax", "sigmoid"],
                 route_norm: bool, route_scale: float, gate_bias: bool,
                 _debug_force_load_balance: bool = False):
        super().__init__()
        self.gate = Linear.Config(bias=gate_bias).build(in_features=dim, out_features=num_experts)
        self.num_experts = num_experts
        self.num_expert_groups = num_expert_groups
        self.num_limited_groups = num_limited_groups
        self.top_k = top_k
        self.score_func = score_func
        self.route_norm = route_norm
        self.route_scale = route_scale
        self._debug_force_load_balance = _debug_force_load_balance

    def _limit_to_groups(self, scores: torch.Tensor) -> torch.Tensor:
        """-inf for the experts of every group outside the `num_limited_groups` best ones, a
        group's score being the sum of its two best experts."""
        if self.num_limited_groups is None:
            raise ValueError("num_limited_groups must be set when num_expert_groups is set")
        if self.num_experts % self.num_expert_groups != 0:
            raise ValueError(f"num_experts ({self.num_experts}) must be divisible by "
                             f"num_expert_groups ({self.num_expert_groups})")
        per_group = self.num_experts // self.num_expert_groups
        if per_group < 2:
            raise ValueError(f"experts_per_group ({per_group}) must be >= 2")
        grouped = scores.view(-1, self.num_expert_groups, per_group)
        group_score = grouped.topk(2, dim=-1).values.sum(dim=-1)
        keep = torch.topk(group_score, k=self.num_limited_groups, dim=-1, sorted=False).indices
        drop = torch.ones_like(group_score, dtype=torch.bool).scatter_(1, keep, False)
        return grouped.masked_fill(drop.unsqueeze(-1), float("-inf")).view(-1, self.num_experts)

    def forward(self, x: torch.Tensor, expert_bias: torch.Tensor | None = None):
        """x [tokens, dim] -> (top_scores [tokens, top_k] float32, expert indices [tokens, top_k],
        tokens per expert [num_experts])."""
        with torch.autocast(device_type=x.device.type, dtype=torch.float32):
            scores = self.gate(x)
        if self.score_func == "sigmoid":
            scores = torch.sigmoid(scores)
        elif self.score_func == "softmax":
            scores = F.softmax(scores, dim=1)
        else:
            raise NotImplementedError(f"Unknown score function {self.score_func}")
        choice = scores if expert_bias is None else scores + expert_bias  # the bias only steers routing
        if self.num_expert_groups is not None:
            choice = self._limit_to_groups(choice)
        selected = torch.topk(choice, k=self.top_k, dim=-1, sorted=False).indices
        top_scores = scores.gather(dim=1, index=selected)
        if self._debug_force_load_balance:  # round-robin assignment, exactly balanced
            n = scores.size(0)
            selected = (torch.arange(n * self.top_k, device=scores.device, dtype=torch.int64)
                        .reshape(n, self.top_k) % self.num_experts)
            top_scores = scores.gather(dim=1, index=selected)
        if self.route_norm:
            top_scores = top_scores / (top_scores.sum(dim=-1, keepdim=True) + 1e-20)
        top_scores = top_scores * self.route_scale
        counts = torch.histc(selected.view(-1), bins=self.num_experts, min=0, max=self.num_experts)
        return top_scores, selected, counts

    def init_weights(self, **kwargs) -> None:
        init_std = kwargs.get("init_std")
        assert init_std is not None
        self.gate.init_weights(init_std=init_std)


class TokenReorderer(Module):
    """Order of the (token, choice) pairs that groups them by expert
    (torchtitan/models/common/moe/moe.py:320-370)."""

    def __init__(self, *, num_experts: int, top_k: int):
        super().__init__()
        self.num_experts = num_experts
        self.top_k = top_k

    def forward(self, top_scores: torch.Tensor, selected_experts_indices: torch.Tensor):
        flat = selected_experts_indices.view(-1)
        counts = torch.histc(flat, bins=self.num_experts, min=0, max=self.num_experts)
        order = torch.argsort(flat, stable=True)
        return top_scores.view(-1)[order], order, counts


class MoE(Module):
    """Router + routed experts (+ shared experts) with auxiliary-loss-free load balancing buffers
    (torchtitan/models/common/moe/moe.py:373-575, single-device part)."""

    @dataclass(kw_only=True, slots=True)
    class Config(Module.Config):
        num_experts: int = 8
        num_shared_experts: int = 1
        score_func: Literal["softmax", "sigmoid"] = "sigmoid"
        route_norm: bool = False
        route_scale: float = 1.0
        gate_bias: bool = False
        score_before_experts: bool = True
        top_k: int = 1
        num_expert_groups: int | None = None
        num_limited_groups: int | None = None
        use_grouped_mm: bool = True
        load_balance_coeff: float | None = 1e-3
        _debug_force_load_balance: bool = False
        hidden_dim: int = 0

    def __init__(self, config: Config, *, dim: int):
        super().__init__()
        self.experts = GroupedExperts(dim=dim, hidden_dim=config.hidden_dim, num_experts=config.num_experts,
                                      use_grouped_mm=config.use_grouped_mm)
        self.router = TokenChoiceTopKRouter(
            dim=dim, num_experts=config.num_experts, num_expert_groups=config.num_expert_groups,
            num_limited_groups=config.num_limited_groups, top_k=config.top_k, score_func=config.score_func,
            route_norm=config.route_norm, route_scale=config.route_scale, gate_bias=config.gate_bias,
            _debug_force_load_balance=config._debug_force_load_balance)
        self.reorderer = TokenReorderer(num_experts=config.num_experts, top_k=config.top_k)
        self.shared_experts = (
            FeedForward.Config(hidden_dim=config.hidden_dim * config.num_shared_experts).build(dim=dim)
            if config.num_shared_experts > 0 else None)
        self.score_before_experts = config.score_before_experts
        self.load_balance_coeff = config.load_balance_coeff
        if self.load_balance_coeff is not None:
            assert self.load_balance_coeff > 0.0
            self.register_buffer("expert_bias", torch.zeros(config.num_experts, dtype=torch.float32), persistent=True)
        else:
            self.expert_bias = None
        self.register_buffer("tokens_per_expert", torch.zeros(config.num_experts, dtype=torch.float32),
                             persistent=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        bs, slen, dim = x.shape
        x = x.view(-1, dim)
        top_scores, selected, counts = self.router(x, self.expert_bias)
        with torch.no_grad():
            self.tokens_per_expert.add_(counts)
        scores_sorted, order, counts = self.reorderer(top_scores, selected)
        top_k = self.router.top_k
        ex = self.experts
        if (ex.use_grouped_mm and x.dtype == torch.bfloat16
                and grouped_feed_forward_fusable(x, ex.w1, ex.w2, ex.w3)
                and ex.w2.mx_config.pad_token_groups_for_grouped_mm):
            # converted experts: gather, score, experts and combine as one fused function
            out_experts = mx_routed_experts(x, top_scores, ex.w1, ex.w2, ex.w3, order, counts,
                                            self.score_before_experts)
            shared = self.shared_experts(x) if self.shared_experts is not None else None
        else:
            routed_in = x[order // top_k]
            if self.score_before_experts:
                routed_in = (routed_in.to(torch.float32) * scores_sorted.reshape(-1, 1)).to(x.dtype)
            routed_out = ex(routed_in, counts)
            shared = self.shared_experts(x) if self.shared_experts is not None else None
            unsorted = torch.zeros((bs * slen * top_k, dim), dtype=routed_out.dtype, device=routed_out.device)
            unsorted[order] = routed_out
            unsorted = unsorted.reshape(-1, top_k, dim)
            if not self.score_before_experts:
                out_experts = torch.bmm(top_scores.reshape(-1, 1, top_k), unsorted.float()).to(x.dtype).squeeze(1)
            else:
                out_experts = unsorted.sum(dim=1)
        if shared is None:
            return out_experts.reshape(bs, slen, dim)
        return (shared + out_experts).reshape(bs, slen, dim)

    def init_weights(self, **kwargs) -> None:
        init_std = kwargs.get("init_std")
        buffer_device = kwargs.get("buffer_device")
        assert init_std is not None
        assert isinstance(buffer_device, torch.device)
        self.experts.init_weights(init_std=init_std)
        self.router.init_weights(init_std=init_std)
        if self.shared_experts is not None:
            self.shared_experts.init_weights(init_std=init_std)
        with torch.device(buffer_device):
            self.tokens_per_expert = torch.zeros(self.experts.num_experts, dtype=torch.float32)
            if self.load_balance_coeff is not None:
                self.expert_bias = torch.zeros(self.experts.num_experts, dtype=torch.float32)
