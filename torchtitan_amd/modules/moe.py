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

from ..mx_tensor import grouped_feed_forward_fusable, mx_grouped_feed_forward
from ..protocols import Module
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
    h = F.silu(torch._grouped_mm(xb, w1.bfloat16().transpose(-2, -1), offs=offsets))
    h = h * torch._grouped_mm(xb, w3.bfloat16().transpose(-2, -1), offs=offsets)
    return torch._grouped_mm(h, w2.bfloat16().transpose(-2, -1), offs=offsets).type_as(x)


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
            if (num_tokens_per_expert.shape[0] == self.w1.shape[0]
                    and grouped_feed_forward_fusable(x, self.w1, self.w2, self.w3)
                    and self.w2.mx_config.pad_token_groups_for_grouped_mm):
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
