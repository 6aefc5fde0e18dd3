"""GPU parity: grouped MXFP8 GEMMs and the token-group padding kernel vs the oracle."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as mo
from tests.helpers import bf16_from_bits, bits_of, randn_bits, rel_l2, u8
from torchtitan_amd import ops

pytestmark = pytest.mark.gpu
TOL = 1e-3
R, L = ops.MX_SCALES_ROWMAJOR, ops.MX_SCALES_MFMA


def _f32(bits):
    return mo.bf16_bits_to_f32(bits)


def _sizes_to_offs(sizes, device):
    return torch.tensor(np.cumsum(sizes), dtype=torch.int32, device=device)


CASES = [
    # (group sizes, N, K)
    ([32, 64, 96], 64, 128),
    ([0, 128, 0, 32], 128, 256),
    ([320, 32, 0, 288, 64], 192, 160),
    ([256, 512, 128], 768, 512),
    ([1024, 96, 608, 0, 32, 992], 256, 384),
]


@pytest.mark.parametrize("sizes,N,K", CASES)
@pytest.mark.parametrize("tail_rows", [0, 64])
def test_grouped_forward_and_dgrad(device, sizes, N, K, tail_rows):
    """2D x 3D: fwd contracts K with W cast along K; dgrad contracts N with W cast along N."""
    rng = np.random.default_rng(sum(sizes) + N + K)
    T = sum(sizes) + tail_rows
    G = len(sizes)
    x_bits = randn_bits(rng, (T, K), outliers=1e-3)
    w_bits = randn_bits(rng, (G, N, K), std=0.02)
    dy_bits = randn_bits(rng, (T, N), std=1e-3)
    offs = _sizes_to_offs(sizes, device)
    x, w, dy = (bf16_from_bits(b, device) for b in (x_bits, w_bits, dy_bits))
    pad64 = N % 128 == 0
    for mode_name, mode in (("floor", mo.FLOOR), ("rceil", mo.RCEIL)):
        wq0, wq1 = ops.to_mx_dim0_dim1_batched(w, mode_name, L)
        if pad64:
            assert torch.equal(wq0.codes, ops.to_mx_dim0_batched(w, mode_name, L).codes)
        y = ops.mx_grouped_gemm_2d3d(ops.to_mx_dim0(x, mode_name, R), wq0, offs)
        ref = mo.grouped_fwd(x_bits, w_bits, np.cumsum(sizes), mode)
        assert rel_l2(_f32(bits_of(y)), _f32(ref)) <= TOL
        assert np.all(bits_of(y)[sum(sizes):] == 0), "padding rows must be zero"
        dx = ops.mx_grouped_gemm_2d3d(ops.to_mx_dim0(dy, mode_name, R), wq1, offs)
        ref = mo.grouped_dgrad(dy_bits, w_bits, np.cumsum(sizes), mode)
        assert rel_l2(_f32(bits_of(dx)), _f32(ref)) <= TOL


@pytest.mark.parametrize("sizes,N,K", CASES)
def test_grouped_wgrad(device, sizes, N, K):
    """2D x 2D: dW[g] contracts the tokens of group g; blocks of 32 run down the tokens."""
    rng = np.random.default_rng(sum(sizes) * 3 + N + K)
    T = sum(sizes) + 32
    x_bits = randn_bits(rng, (T, K), outliers=1e-3)
    dy_bits = randn_bits(rng, (T, N), std=1e-3)
    offs = _sizes_to_offs(sizes, device)
    x, dy = bf16_from_bits(x_bits, device), bf16_from_bits(dy_bits, device)
    for mode_name, mode in (("floor", mo.FLOOR), ("rceil", mo.RCEIL)):
        dw = ops.mx_grouped_gemm_2d2d(ops.to_mx_dim1(dy, mode_name, R), ops.to_mx_dim1(x, mode_name, R), offs)
        ref = mo.grouped_wgrad(dy_bits, x_bits, np.cumsum(sizes), mode)
        got = bits_of(dw)
        for g, s in enumerate(sizes):
            if s == 0:
                assert np.all(got[g] == 0)
            else:
                assert rel_l2(_f32(got[g]), _f32(ref[g])) <= TOL, g


FAST_CASES = [
    # (group sizes, multiples of 32; N; K) -- the persistent-kernel forms (MFMA-order scales)
    ([128, 256, 384], 256, 128),
    ([0, 128, 0, 640, 0], 128, 256),
    ([512, 128, 0, 1024, 256], 768, 384),
    ([1280, 384], 264, 512),
    # groups that start and end inside 128-row scale groups / 128-deep K blocks
    ([96, 160, 32, 0, 416, 288], 256, 256),
    ([32, 32, 32, 32, 32, 1056, 64], 384, 128),
    ([352, 2880, 0, 64, 992], 256, 384),
    ([224, 0, 0, 32, 608, 96, 320], 520, 256),
]


@pytest.mark.parametrize("sizes,N,K", FAST_CASES)
@pytest.mark.parametrize("tail_rows", [0, 128, 384])
def test_grouped_forward_and_dgrad_aligned_groups(device, sizes, N, K, tail_rows):
    """2D x 3D through the persistent kernel: groups end at multiples of 32, MFMA-order scales."""
    rng = np.random.default_rng(sum(sizes) + N + K + 7)
    T = sum(sizes) + tail_rows
    G = len(sizes)
    x_bits = randn_bits(rng, (T, K), outliers=1e-3)
    w_bits = randn_bits(rng, (G, N, K), std=0.02)
    offs = _sizes_to_offs(sizes, device)
    x, w = bf16_from_bits(x_bits, device), bf16_from_bits(w_bits, device)
    for mode_name, mode in (("floor", mo.FLOOR), ("rceil", mo.RCEIL)):
        wq0 = ops.to_mx_dim0_batched(w, mode_name, L)
        y = ops.mx_grouped_gemm_2d3d(ops.to_mx_dim0(x, mode_name, L), wq0, offs)
        ref = mo.grouped_fwd(x_bits, w_bits, np.cumsum(sizes), mode)
        assert rel_l2(_f32(bits_of(y)), _f32(ref)) <= TOL
        assert np.all(bits_of(y)[sum(sizes):] == 0), "rows behind the last group must be zero"
        # the general kernel (row-major scales) must agree to the last bit on the same operands
        y2 = ops.mx_grouped_gemm_2d3d(ops.to_mx_dim0(x, mode_name, R), wq0, offs)
        assert rel_l2(_f32(bits_of(y)), _f32(bits_of(y2))) <= 2e-3
    if N % 128 == 0:
        dy_bits = randn_bits(rng, (T, N), std=1e-3)
        dy = bf16_from_bits(dy_bits, device)
        wq1 = ops.to_mx_dim1_batched(w, "rceil", L)
        dx = ops.mx_grouped_gemm_2d3d(ops.to_mx_dim0(dy, "rceil", L), wq1, offs)
        ref = mo.grouped_dgrad(dy_bits, w_bits, np.cumsum(sizes), mo.RCEIL)
        assert rel_l2(_f32(bits_of(dx)), _f32(ref)) <= TOL


@pytest.mark.parametrize("sizes,N,K", FAST_CASES)
def test_grouped_wgrad_aligned_groups(device, sizes, N, K):
    """2D x 2D through the persistent kernel: token groups end at multiples of 32 (the token axis
    itself is a multiple of 128 and runs past the last group)."""
    rng = np.random.default_rng(sum(sizes) * 5 + N + K)
    T = -(-(sum(sizes) + 128) // 128) * 128
    x_bits = randn_bits(rng, (T, K), outliers=1e-3)
    dy_bits = randn_bits(rng, (T, N), std=1e-3)
    offs = _sizes_to_offs(sizes, device)
    x, dy = bf16_from_bits(x_bits, device), bf16_from_bits(dy_bits, device)
    for mode_name, mode in (("floor", mo.FLOOR), ("rceil", mo.RCEIL)):
        dw = ops.mx_grouped_gemm_2d2d(ops.to_mx_dim1(dy, mode_name, L), ops.to_mx_dim1(x, mode_name, L), offs)
        ref = mo.grouped_wgrad(dy_bits, x_bits, np.cumsum(sizes), mode)
        got = bits_of(dw)
        for g, s_ in enumerate(sizes):
            if s_ == 0:
                assert np.all(got[g] == 0)
            else:
                assert rel_l2(_f32(got[g]), _f32(ref[g])) <= TOL, g


def test_aligned_group_forms_split_into_several_launches(device):
    """More tiles than a workgroup can keep records for: the launch is cut by tile columns.

    Forced here by running with 8 workgroups (a debug setting of the library), which lowers the
    capacity of one launch to 952 tiles."""
    from torchtitan_amd import _lib

    lib = _lib.load()
    rng = np.random.default_rng(23)
    try:
        lib.mx_debug_set_grid(8)
        sizes, N, K = [512, 0, 1280], 25600, 128      # 12 tile rows x 100 tile columns
        T = sum(sizes) + 256
        x_bits = randn_bits(rng, (T, K), outliers=1e-3)
        w_bits = randn_bits(rng, (len(sizes), N, K), std=0.02)
        offs = _sizes_to_offs(sizes, device)
        x, w = bf16_from_bits(x_bits, device), bf16_from_bits(w_bits, device)
        y = ops.mx_grouped_gemm_2d3d(ops.to_mx_dim0(x, "rceil", L), ops.to_mx_dim0_batched(w, "rceil", L), offs)
        ref = mo.grouped_fwd(x_bits, w_bits, np.cumsum(sizes), mo.RCEIL)
        assert rel_l2(_f32(bits_of(y)), _f32(ref)) <= TOL
        assert np.all(bits_of(y)[sum(sizes):] == 0)

        sizes, N, K = [128, 0, 256], 2560, 10240      # 30 tiles per column x 40 tile columns
        T = sum(sizes)
        x_bits = randn_bits(rng, (T, K), outliers=1e-3)
        dy_bits = randn_bits(rng, (T, N), std=1e-3)
        offs = _sizes_to_offs(sizes, device)
        x, dy = bf16_from_bits(x_bits, device), bf16_from_bits(dy_bits, device)
        dw = ops.mx_grouped_gemm_2d2d(ops.to_mx_dim1(dy, "rceil", L), ops.to_mx_dim1(x, "rceil", L), offs)
        ref = mo.grouped_wgrad(dy_bits, x_bits, np.cumsum(sizes), mo.RCEIL)
        got = bits_of(dw)
        assert np.all(got[1] == 0)
        for g in (0, 2):
            assert rel_l2(_f32(got[g]), _f32(ref[g])) <= TOL, g
    finally:
        lib.mx_debug_set_grid(0)


def test_neighbouring_groups_do_not_leak_into_a_ragged_group(device):
    """A group that ends inside a 128-row scale group / a 128-deep K block shares that block with
    its neighbour in memory.  NaN everywhere in the neighbours must not reach its results."""
    rng = np.random.default_rng(77)
    sizes, N, K = [160, 96, 224, 32], 256, 256    # ends 160, 256, 480, 512
    T = sum(sizes)
    x_bits = randn_bits(rng, (T, K), outliers=1e-3)
    dy_bits = randn_bits(rng, (T, N), std=1e-3)
    w_bits = randn_bits(rng, (len(sizes), N, K), std=0.02)
    lo, hi = 256, 480                               # group 2
    x_nan, dy_nan = x_bits.copy(), dy_bits.copy()
    x_nan[:lo] = 0x7FC0
    x_nan[hi:] = 0x7FC0
    dy_nan[:lo] = 0x7FC0
    dy_nan[hi:] = 0x7FC0
    offs = _sizes_to_offs(sizes, device)
    x, dy, w = bf16_from_bits(x_nan, device), bf16_from_bits(dy_nan, device), bf16_from_bits(w_bits, device)
    y = ops.mx_grouped_gemm_2d3d(ops.to_mx_dim0(x, "rceil", L), ops.to_mx_dim0_batched(w, "rceil", L), offs)
    ref = mo.grouped_fwd(x_bits, w_bits, np.cumsum(sizes), mo.RCEIL)
    assert rel_l2(_f32(bits_of(y)[lo:hi]), _f32(ref[lo:hi])) <= TOL
    assert torch.isnan(y[:lo]).all() and torch.isnan(y[hi:]).all()
    dw = ops.mx_grouped_gemm_2d2d(ops.to_mx_dim1(dy, "rceil", L), ops.to_mx_dim1(x, "rceil", L), offs)
    refw = mo.grouped_wgrad(dy_bits, x_bits, np.cumsum(sizes), mo.RCEIL)
    assert rel_l2(_f32(bits_of(dw)[2]), _f32(refw[2])) <= TOL
    assert torch.isnan(dw[0]).all() and torch.isnan(dw[1]).all() and torch.isnan(dw[3]).all()


def test_aligned_group_forms_poison_the_output_when_a_group_end_is_not_a_multiple_of_32(device):
    rng = np.random.default_rng(5)
    sizes, N, K = [128, 144, 112], 128, 128
    T = sum(sizes)
    x = bf16_from_bits(randn_bits(rng, (T, K)), device)
    w = bf16_from_bits(randn_bits(rng, (len(sizes), N, K), std=0.02), device)
    offs = _sizes_to_offs(sizes, device)
    y = ops.mx_grouped_gemm_2d3d(ops.to_mx_dim0(x, "rceil", L), ops.to_mx_dim0_batched(w, "rceil", L), offs)
    assert torch.isnan(y).all()
    dy = bf16_from_bits(randn_bits(rng, (T, N), std=1e-3), device)
    dw = ops.mx_grouped_gemm_2d2d(ops.to_mx_dim1(dy, "rceil", L), ops.to_mx_dim1(x, "rceil", L), offs)
    assert torch.isnan(dw).all()


def test_row_major_wgrad_poisons_groups_that_break_the_32_token_rule(device):
    """Row-major scales: a group may be any multiple of 32 tokens.  A group that starts or ends
    inside a 32-token block would share scale blocks with its neighbour; its weight gradient
    comes out as NaN, the groups that keep the rule are still right."""
    rng = np.random.default_rng(8)
    sizes, N, K = [64, 40, 56, 96], 160, 96   # ends 64, 104, 160, 256: groups 1 and 2 touch 104
    T = sum(sizes)
    x_bits, dy_bits = randn_bits(rng, (T, K)), randn_bits(rng, (T, N), std=1e-3)
    x, dy = bf16_from_bits(x_bits, device), bf16_from_bits(dy_bits, device)
    offs = _sizes_to_offs(sizes, device)
    dw = ops.mx_grouped_gemm_2d2d(ops.to_mx_dim1(dy, "rceil", R), ops.to_mx_dim1(x, "rceil", R), offs)
    assert torch.isnan(dw[1]).all() and torch.isnan(dw[2]).all()
    lo = 0
    for g, n in enumerate(sizes):
        if g in (0, 3):
            ref = mo.mx_matmul(np.ascontiguousarray(dy_bits[lo:lo + n].T), np.ascontiguousarray(x_bits[lo:lo + n].T), mo.RCEIL)
            assert rel_l2(_f32(bits_of(dw[g])), _f32(ref)) <= TOL, g
        lo += n


def test_batched_weight_casts_match_per_matrix(device):
    rng = np.random.default_rng(11)
    w_bits = randn_bits(rng, (5, 96, 160), std=0.02, outliers=1e-3)
    w = bf16_from_bits(w_bits, device)
    for order in (R, L):
        q0, q1 = ops.to_mx_dim0_dim1_batched(w, "rceil", order)
        q1b = ops.to_mx_dim1_batched(w, "rceil", order)
        assert torch.equal(q1.codes, q1b.codes) and torch.equal(q1.scales.reshape(-1), q1b.scales.reshape(-1))
        for g in range(5):
            c0, s0 = mo.cast_dim0(w_bits[g], mo.RCEIL)
            c1, s1 = mo.cast_dim1(w_bits[g], mo.RCEIL)
            assert np.array_equal(u8(q0.codes[g]), c0) and np.array_equal(u8(q1.codes[g]), c1)
            if order == L:
                s0, s1 = mo.scale_layout(s0).reshape(-1), mo.scale_layout(s1).reshape(-1)
                n0, n1 = s0.size, s1.size
                assert np.array_equal(u8(q0.scales)[g * n0:(g + 1) * n0], s0)
                assert np.array_equal(u8(q1.scales)[g * n1:(g + 1) * n1], s1)
            else:
                assert np.array_equal(u8(q0.scales[g]), s0) and np.array_equal(u8(q1.scales[g]), s1)


# ---------------------------------------------------------------- padding / permutation
def _check_pad(device, counts, experts, ranks, alignment, max_len):
    perm, m_sizes, m_offsets = ops.group_offsets_pad(torch.tensor(counts, device=device), experts, ranks, max_len, alignment)
    rp, rs, ro = mo.generate_permute_indices(np.asarray(counts), experts, ranks, max_len, alignment)
    assert np.array_equal(perm.cpu().numpy(), rp)
    assert np.array_equal(m_sizes.cpu().numpy(), rs) and m_sizes.dtype == torch.int32
    assert np.array_equal(m_offsets.cpu().numpy(), ro) and m_offsets.dtype == torch.int32


def test_pad_docstring_example(device):
    # the worked example of generate_permute_indices: 2 ranks x 4 experts
    _check_pad(device, [4, 2, 1, 3, 1, 2, 3, 4], 4, 2, 8, mo.padded_max_len(20, 4, 8))


@pytest.mark.parametrize("ranks", [1, 2, 4, 8, 16])
@pytest.mark.parametrize("token_range", [(1, 16), (0, 5), (0, 0), (100, 2000)])
def test_pad_matches_reference_fill(device, ranks, token_range):
    rng = np.random.default_rng(2020 + ranks)
    total_experts = 256
    experts = total_experts // ranks
    counts = rng.integers(token_range[0], token_range[1] + 1, size=total_experts).tolist()
    for alignment in (8, 16, 32):
        max_len = mo.padded_max_len(sum(counts), experts, alignment)
        _check_pad(device, counts, experts, ranks, alignment, max_len)
        _check_pad(device, counts, experts, ranks, alignment, max(sum(counts) // 2, 1))  # truncated


def test_pad_then_grouped_gemm_moe_like(device):
    """Routed tokens -> padded groups -> grouped GEMM, against the per-expert oracle loop."""
    rng = np.random.default_rng(5)
    E, dim, hidden, A = 8, 256, 192, 32
    counts = np.array([37, 0, 130, 64, 1, 95, 0, 200])
    T = int(counts.sum())
    x_bits = randn_bits(rng, (T, dim))
    w_bits = randn_bits(rng, (E, hidden, dim), std=0.02)
    max_len = mo.padded_max_len(T, E, A)
    perm, m_sizes, m_offsets = ops.group_offsets_pad(torch.tensor(counts, device=device), E, 1, max_len, A)
    x = bf16_from_bits(x_bits, device)
    xp = torch.vstack((x, x.new_zeros((1, dim))))[perm]
    y = ops.mx_grouped_gemm_2d3d(ops.to_mx_dim0(xp, "rceil", R), ops.to_mx_dim0_batched(bf16_from_bits(w_bits, device), "rceil", L), m_offsets)
    rp, rs, ro = mo.generate_permute_indices(counts, E, 1, max_len, A)
    xp_bits = np.vstack((x_bits, np.zeros((1, dim), np.uint16)))[rp]
    ref = mo.grouped_fwd(xp_bits, w_bits, ro, mo.RCEIL)
    assert rel_l2(_f32(bits_of(y)), _f32(ref)) <= TOL


@pytest.mark.parametrize("experts,top_k,tokens,align", [(4, 2, 50, 32), (16, 4, 300, 128), (128, 8, 2048, 128)])
def test_moe_route_plan_matches_the_oracle(device, experts, top_k, tokens, align):
    """One-launch routing plan (padded group ends, token and score of every padded row, padded
    row of every pair) against the oracle's composition of the padding rule with the sorted
    order; integer outputs and copied scores: exact.  One expert left without tokens."""
    rng = np.random.default_rng(experts + tokens)
    choice = rng.integers(0, experts - 1, (tokens, top_k))     # the last expert stays empty
    order = np.argsort(choice.reshape(-1), kind="stable").astype(np.int64)
    counts = np.bincount(choice.reshape(-1), minlength=experts).astype(np.int32)
    scores = rng.random(tokens * top_k).astype(np.float32)
    offs, src_row, row_score, pos = ops.moe_route_plan(
        torch.from_numpy(counts).to(device), torch.from_numpy(order).to(device),
        torch.from_numpy(scores).to(device), top_k, align)
    o_offs, o_src, o_score, o_pos = mo.moe_route_plan(counts, order, scores, top_k, align)
    assert np.array_equal(offs.cpu().numpy(), o_offs)
    assert np.array_equal(src_row.cpu().numpy(), o_src)
    assert np.array_equal(row_score.cpu().numpy(), o_score)
    assert np.array_equal(pos.cpu().numpy(), o_pos)
    # the plan is a bijection between pairs and non-padding rows, grouped by expert
    valid = o_src >= 0
    assert valid.sum() == tokens * top_k and np.array_equal(np.sort(o_pos), np.nonzero(valid)[0])
    ends = np.concatenate(([0], o_offs))
    for e in range(experts):
        rows = np.nonzero(valid[ends[e]:ends[e + 1]])[0]
        assert len(rows) == counts[e] and (len(rows) == 0 or rows[-1] == len(rows) - 1)


@pytest.mark.parametrize("align", [32, 128])
def test_moe_config_full_size_groups_equal_dense_gemms(device, align):
    """The MoE configuration at full size (128 experts, dim 2048, expert FFN 768, 16384 tokens x
    top-8 = 131 072 routed rows, group sizes from a softmax over seeded Gumbel-perturbed logits,
    groups padded to multiples of 32 rows as the configuration says, or of 128): no oracle at this
    size, but a grouped GEMM is a stack of dense ones.  For the smallest, the largest and two
    other experts the group's rows of the forward and dgrad outputs are bit-identical to the
    dense kernel on that group's operands alone (same codes, same K order), and so is its weight
    gradient when the group is whole 128-deep blocks (otherwise the dense call runs on another
    kernel with another summation order: rel-L2); rows behind the last group are zero."""
    E, D, H, tokens, top_k = 128, 2048, 768, 16384, 8
    torch.manual_seed(4)
    logits = torch.randn(tokens, E, device=device) + 0.5 * torch.randn(E, device=device)
    gumbel = -torch.log(-torch.log(torch.rand(tokens, E, device=device).clamp_min(1e-9)))
    picked = torch.topk(torch.softmax(logits + gumbel, dim=-1), top_k, dim=-1).indices
    counts = torch.bincount(picked.flatten(), minlength=E)
    sizes = ((counts + align - 1) // align * align).cpu().numpy()
    assert counts.sum() == tokens * top_k and sizes.min() != sizes.max()
    if align == 32:
        assert any(int(v) % 128 for v in sizes) and any(int(e) % 128 for e in np.cumsum(sizes))
    ends = np.cumsum(sizes)
    Tp = -(-(int(ends[-1]) + 256) // 128) * 128  # at least two tiles' worth of rows that belong to no expert
    offs = _sizes_to_offs(sizes, device)
    x = torch.randn(Tp, D, device=device, dtype=torch.bfloat16)
    dy = torch.randn(Tp, H, device=device, dtype=torch.bfloat16) * 1e-3
    w = torch.randn(E, H, D, device=device, dtype=torch.bfloat16) * 0.02
    xq0, xq1 = ops.to_mx_dim0_dim1(x, "rceil", L)
    dyq0, dyq1 = ops.to_mx_dim0_dim1(dy, "rceil", L)
    wq0, wq1 = ops.to_mx_dim0_dim1_batched(w, "rceil", L)
    y = ops.mx_grouped_gemm_2d3d(xq0, wq0, offs)        # [Tp, H]
    dx = ops.mx_grouped_gemm_2d3d(dyq0, wq1, offs)      # [Tp, D]
    dw = ops.mx_grouped_gemm_2d2d(dyq1, xq1, offs)      # [E, H, D]
    assert not bool(y[int(ends[-1]):].any()) and not bool(dx[int(ends[-1]):].any())
    assert not bool(torch.isnan(y).any() | torch.isnan(dx).any()) and not bool(torch.isnan(dw).any())
    from torchtitan_amd import _lib

    order = np.argsort(sizes)
    _lib.load().mx_debug_force_kernel(3)  # the dense calls on the same (persistent) kernel
    try:
        for g in (int(order[0]), int(order[-1]), int(order[E // 2]), E - 1):
            lo, hi = int(ends[g] - sizes[g]), int(ends[g])
            xg, dyg = x[lo:hi].contiguous(), dy[lo:hi].contiguous()
            xg0, xg1 = ops.to_mx_dim0_dim1(xg, "rceil", L)
            dyg0, dyg1 = ops.to_mx_dim0_dim1(dyg, "rceil", L)
            wg0, wg1 = ops.to_mx_dim0_dim1(w[g].contiguous(), "rceil", L)
            assert torch.equal(y[lo:hi], ops.mx_gemm_nt(xg0, wg0)), g
            assert torch.equal(dx[lo:hi], ops.mx_gemm_nt(dyg0, wg1)), g
            dwg = ops.mx_gemm_nt(dyg1, xg1)
            if (hi - lo) % 128 == 0:
                assert torch.equal(dw[g], dwg), g
            else:
                assert rel_l2(dw[g].float().cpu().numpy(), dwg.float().cpu().numpy()) <= TOL, g
    finally:
        _lib.load().mx_debug_force_kernel(0)


@pytest.mark.parametrize("G,N,K", [(40, 256, 512), (33, 512, 256), (67, 384, 256)])
def test_grouped_wgrad_many_uneven_groups(device, G, N, K):
    """From 32 groups on the persistent wgrad kernel deals its tiles by group length (longest
    first, back and forth over XCDs and workgroups) instead of in tile order: every group's
    gradient against the oracle, with empty groups, one long group and a tail that belongs to
    no group."""
    rng = np.random.default_rng(G * 13 + N + K)
    sizes = rng.choice([0, 128, 128, 256, 384, 640], size=G).tolist()
    sizes[G // 2] = 1536
    sizes[3] = 0
    T = sum(sizes) + 256
    x_bits = randn_bits(rng, (T, K), outliers=1e-3)
    dy_bits = randn_bits(rng, (T, N), std=1e-3)
    offs = _sizes_to_offs(sizes, device)
    x, dy = bf16_from_bits(x_bits, device), bf16_from_bits(dy_bits, device)
    dw = ops.mx_grouped_gemm_2d2d(ops.to_mx_dim1(dy, "rceil", L), ops.to_mx_dim1(x, "rceil", L), offs)
    ref = mo.grouped_wgrad(dy_bits, x_bits, np.cumsum(sizes), mo.RCEIL)
    got = bits_of(dw)
    for g, s_ in enumerate(sizes):
        if s_ == 0:
            assert np.all(got[g] == 0), g
        else:
            assert rel_l2(_f32(got[g]), _f32(ref[g])) <= TOL, g


@pytest.mark.parametrize("sizes,N,K,tail", [([256, 0, 128, 640], 256, 256, 128), ([128] * 9 + [1024, 0, 384], 512, 384, 0)])
def test_grouped_pair_gemm_matches_the_oracle_over_the_concatenated_contraction(device, sizes, N, K, tail):
    """Two operand sets summed per output tile in the grouped 2D x 3D kernel: against the oracle's
    grouped forward of [X | X2] with [W | W2] (contraction 2K), rows behind the last group zero."""
    rng = np.random.default_rng(sum(sizes) + N + K)
    T, G = sum(sizes) + tail, len(sizes)
    x_bits, x2_bits = randn_bits(rng, (T, K)), randn_bits(rng, (T, K), std=0.3)
    w_bits, w2_bits = randn_bits(rng, (G, N, K), std=0.02), randn_bits(rng, (G, N, K), std=0.05)
    offs = _sizes_to_offs(sizes, device)
    q = lambda bits: ops.to_mx_dim0(bf16_from_bits(bits, device), "rceil", L)
    qb = lambda bits: ops.to_mx_dim0_batched(bf16_from_bits(bits, device), "rceil", L)
    launches = []
    real_call = ops._call
    ops._call = lambda name, *rest: (launches.append(name), real_call(name, *rest))[1]
    try:
        y = ops.mx_grouped_gemm_2d3d_pair(q(x_bits), qb(w_bits), q(x2_bits), qb(w2_bits), offs)
    finally:
        ops._call = real_call
    assert "mx_grouped_gemm_2d3d_pair" in launches
    ref = mo.grouped_fwd(np.concatenate([x_bits, x2_bits], 1), np.concatenate([w_bits, w2_bits], 2),
                         np.cumsum(sizes), mo.RCEIL)
    assert rel_l2(_f32(bits_of(y)), _f32(ref)) <= TOL
    assert np.all(bits_of(y)[sum(sizes):] == 0)


def _launch_names(fn):
    names = []
    real_call = ops._call
    ops._call = lambda name, *rest: (names.append(name), real_call(name, *rest))[1]
    try:
        return fn(), names
    finally:
        ops._call = real_call


@pytest.mark.parametrize("sizes,N,K,tail", [([256, 0, 128, 640], 256, 256, 128), ([96, 160, 32, 0, 416, 288], 264, 384, 0),
                                            ([128] * 9 + [1024, 0, 384], 768, 512, 256)])
def test_grouped_forward_of_two_weight_stacks_in_one_launch(device, sizes, N, K, tail):
    """x against w1[g] and w3[g] in one launch of the persistent kernel: both outputs bit-identical
    to the two separate grouped GEMMs (ragged 32-aligned groups, rows behind the last group zero)."""
    rng = np.random.default_rng(sum(sizes) + N + K + 1)
    T, G = sum(sizes) + tail, len(sizes)
    offs = _sizes_to_offs(sizes, device)
    xq = ops.to_mx_dim0(bf16_from_bits(randn_bits(rng, (T, K), outliers=1e-3), device), "rceil", L)
    w1 = ops.to_mx_dim0_batched(bf16_from_bits(randn_bits(rng, (G, N, K), std=0.02), device), "rceil", L)
    w3 = ops.to_mx_dim0_batched(bf16_from_bits(randn_bits(rng, (G, N, K), std=0.05), device), "rceil", L)
    (h1, h3), names = _launch_names(lambda: ops.mx_grouped_gemm_2d3d_shared_a(xq, w1, w3, offs))
    assert names == ["mx_grouped_gemm_2d3d_shared_a"]
    assert torch.equal(h1, ops.mx_grouped_gemm_2d3d(xq, w1, offs))
    assert torch.equal(h3, ops.mx_grouped_gemm_2d3d(xq, w3, offs))
    assert not h1[sum(sizes):].any() and not h3[sum(sizes):].any()
    # a broken group end poisons both outputs
    bad = offs.clone()
    bad[0] += 8
    p1, p3 = ops.mx_grouped_gemm_2d3d_shared_a(xq, w1, w3, bad)
    assert p1.isnan().all() and p3.isnan().all()


@pytest.mark.parametrize("sizes,N,K", [([256, 0, 128, 640], 256, 256), ([96, 160, 32, 0, 416, 288], 264, 384),
                                       ([32 * (1 + (7 * g) % 11) for g in range(40)], 768, 512)])
def test_grouped_wgrads_of_two_gradients_in_one_launch(device, sizes, N, K):
    """da^T x and db^T x per group in one launch: bit-identical to the two separate 2D x 2D GEMMs,
    also with enough groups for the dealing of tiles by group length."""
    rng = np.random.default_rng(sum(sizes) * 3 + N + K)
    T = -(-(sum(sizes) + 128) // 128) * 128
    offs = _sizes_to_offs(sizes, device)
    col = lambda cols, std: ops.to_mx_dim1(bf16_from_bits(randn_bits(rng, (T, cols), std=std), device), "rceil", L)
    da, db, x = col(N, 1e-3), col(N, 3e-3), col(K, 1.0)
    (dw1, dw3), names = _launch_names(lambda: ops.mx_grouped_gemm_2d2d_shared_b(da, db, x, offs))
    assert names == ["mx_grouped_gemm_2d2d_shared_b"]
    assert torch.equal(dw1, ops.mx_grouped_gemm_2d2d(da, x, offs))
    assert torch.equal(dw3, ops.mx_grouped_gemm_2d2d(db, x, offs))


@pytest.mark.parametrize("real,N,K,tail_p,tail_out,two", [
    ([250, 0, 97, 640, 1], 256, 256, 128, 0, False),     # ragged real sizes, an empty group, a one-row group
    ([250, 0, 97, 640, 1], 264, 384, 128, 5, True),      # rows that belong to no group: zeros
    ([300] * 3 + [31, 33, 1000, 0, 511], 768, 512, 256, 0, True),  # groups over several tiles
])
def test_grouped_gemm_leaves_the_padding_out_of_its_output(device, real, N, K, tail_p, tail_out, two):
    """mx_grouped_gemm_2d3d_rows_out (one product and the sum of two): bit-identical to the grouped
    GEMM over the padded groups followed by the gather of the real rows; rows of the output behind
    the last group are zero, a row next to the output is not touched, and a broken (padded) group
    end poisons exactly the output's rows."""
    rng = np.random.default_rng(sum(real) + N + K + int(two))
    G = len(real)
    padded = [-(-r // 32) * 32 if r else 32 * (g % 2) for g, r in enumerate(real)]  # some empty groups get a block
    Tp = sum(padded) + tail_p
    T = sum(real) + tail_out
    offs_p = _sizes_to_offs(padded, device)
    offs = _sizes_to_offs(real, device)
    q = lambda std: ops.to_mx_dim0(bf16_from_bits(randn_bits(rng, (Tp, K), std=std, outliers=1e-3), device), "rceil", L)
    qb = lambda std: ops.to_mx_dim0_batched(bf16_from_bits(randn_bits(rng, (G, N, K), std=std), device), "rceil", L)
    a, b = q(1.0), qb(0.02)
    a2, b2 = (q(0.3), qb(0.05)) if two else (None, None)
    full = ops.mx_grouped_gemm_2d3d_pair(a, b, a2, b2, offs_p) if two else ops.mx_grouped_gemm_2d3d(a, b, offs_p)
    # the rows a gather would take: the first real[g] rows of padded group g, then zero rows
    starts_p = np.cumsum([0] + padded[:-1])
    rows = np.concatenate([np.arange(s, s + r) for s, r in zip(starts_p, real)] + [np.full(tail_out, -1)]).astype(np.int64)
    idx = torch.from_numpy(rows).to(device)
    want = torch.where((idx >= 0)[:, None], full[idx.clamp_min(0)], torch.zeros((), dtype=full.dtype, device=device))
    got, names = _launch_names(lambda: ops.mx_grouped_gemm_2d3d_rows_out(a, b, offs_p, offs, T, a2, b2))
    assert names == ["mx_grouped_gemm_2d3d_rows_out"]
    assert got.shape == (T, N) and torch.equal(got, want)
    # through the C ABI into a buffer with a guard row on each side and a wider row pitch
    from torchtitan_amd import _lib
    ld = N + 8
    buf = torch.full((T + 2, ld), 7.0, dtype=torch.bfloat16, device=device)
    second = [ops._ptr(t) for t in (a2.codes, a2.scales, b2.codes, b2.scales)] if two else [None] * 4
    st = _lib.load().mx_grouped_gemm_2d3d_rows_out(
        ops._ptr(a.codes), ops._ptr(a.scales), ops._ptr(b.codes), ops._ptr(b.scales), *second, ops._ptr(offs_p),
        ops._ptr(offs), ops._ptr(buf[1]), Tp, T, N, K, G, ld, ops._stream(buf))
    assert st == 0
    assert torch.equal(buf[1:T + 1, :N], want)
    assert (buf[0] == 7).all() and (buf[T + 1] == 7).all() and (buf[:, N:] == 7).all()
    # a padded group end that is no multiple of 32: NaN over the output, nothing beyond it
    bad = offs_p.clone()
    bad[0] += 8
    buf.fill_(7.0)
    st = _lib.load().mx_grouped_gemm_2d3d_rows_out(
        ops._ptr(a.codes), ops._ptr(a.scales), ops._ptr(b.codes), ops._ptr(b.scales), *second, ops._ptr(bad),
        ops._ptr(offs), ops._ptr(buf[1]), Tp, T, N, K, G, ld, ops._stream(buf))
    assert st == 0
    assert buf[1:T + 1, :N].isnan().all()
    assert (buf[0] == 7).all() and (buf[T + 1] == 7).all() and (buf[:, N:] == 7).all()
    # unpadded group ends that make no sense never reach outside the output
    wild = torch.tensor([-5, 10 ** 6] + [T // 2] * (G - 2), dtype=torch.int32, device=device)[:G]
    buf.fill_(7.0)
    st = _lib.load().mx_grouped_gemm_2d3d_rows_out(
        ops._ptr(a.codes), ops._ptr(a.scales), ops._ptr(b.codes), ops._ptr(b.scales), *second, ops._ptr(offs_p),
        ops._ptr(wild), ops._ptr(buf[1]), Tp, T, N, K, G, ld, ops._stream(buf))
    assert st == 0
    assert (buf[0] == 7).all() and (buf[T + 1] == 7).all() and (buf[:, N:] == 7).all()
    # bad arguments
    assert _lib.load().mx_grouped_gemm_2d3d_rows_out(
        ops._ptr(a.codes), ops._ptr(a.scales), ops._ptr(b.codes), ops._ptr(b.scales), *second, ops._ptr(offs_p),
        ops._ptr(offs), ops._ptr(buf[1]), Tp, Tp + 1, N, K, G, ld, ops._stream(buf)) != 0
