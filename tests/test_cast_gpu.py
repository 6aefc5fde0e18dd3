"""GPU parity: HIP to_mx casts vs the CPU oracle, bit-exact (codes and scale bytes)."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as mo
from tests.helpers import bf16_from_bits, bits_of, randn_bits, u8
from torchtitan_amd import _lib, ops

pytestmark = pytest.mark.gpu

MODES = [("floor", mo.FLOOR), ("rceil", mo.RCEIL)]


def _check_dim0(bits, mode_name, mode, device):
    x = bf16_from_bits(bits, device)
    got = ops.to_mx_dim0(x, mode_name)
    codes, scales = mo.cast_dim0(bits, mode)
    assert np.array_equal(u8(got.scales), scales), "scale bytes differ"
    assert np.array_equal(u8(got.codes), codes), "codes differ"
    laid = ops.to_mx_dim0(x, mode_name, ops.MX_SCALES_MFMA)
    assert np.array_equal(u8(laid.codes), codes)
    assert np.array_equal(u8(laid.scales).reshape(-1), mo.scale_layout(scales).reshape(-1))


def _check_dim1(bits, mode_name, mode, device):
    x = bf16_from_bits(bits, device)
    got = ops.to_mx_dim1(x, mode_name)
    codes, scales = mo.cast_dim1(bits, mode)
    assert np.array_equal(u8(got.scales), scales), "scale bytes differ"
    assert np.array_equal(u8(got.codes), codes), "codes differ"
    laid = ops.to_mx_dim1(x, mode_name, ops.MX_SCALES_MFMA)
    assert np.array_equal(u8(laid.codes), codes)
    assert np.array_equal(u8(laid.scales).reshape(-1), mo.scale_layout(scales).reshape(-1))


def _check_fused(bits, mode_name, mode, device):
    x = bf16_from_bits(bits, device)
    for order in (ops.MX_SCALES_ROWMAJOR, ops.MX_SCALES_MFMA):
        r, c = ops.to_mx_dim0_dim1(x, mode_name, order)
        c0, s0 = mo.cast_dim0(bits, mode)
        c1, s1 = mo.cast_dim1(bits, mode)
        if order == ops.MX_SCALES_MFMA:
            s0, s1 = mo.scale_layout(s0).reshape(-1), mo.scale_layout(s1).reshape(-1)
        assert np.array_equal(u8(r.codes), c0) and np.array_equal(u8(c.codes), c1)
        assert np.array_equal(u8(r.scales).reshape(-1), s0.reshape(-1))
        assert np.array_equal(u8(c.scales).reshape(-1), s1.reshape(-1))


@pytest.mark.parametrize("mode_name,mode", MODES)
def test_every_bf16_value_as_amax_dim0(device, mode_name, mode):
    """All 65536 bf16 patterns as the first lane of a block, three fill patterns for the rest."""
    allv = np.arange(65536, dtype=np.uint16)
    rng = np.random.default_rng(0)
    for fill in ("zero", "half", "random"):
        blk = np.zeros((65536, 32), dtype=np.uint16)
        blk[:, 0] = allv
        if fill == "half":  # other lanes: amax / 2 with alternating sign (exponent - 1)
            e = (allv >> 7) & 0xFF
            half = np.where(e > 1, allv - np.uint16(0x80), np.uint16(0)) & np.uint16(0x7FFF)
            half = np.where((allv & 0x7FFF) > 0x7F80, np.uint16(0x3F80), half)
            blk[:, 1:] = half[:, None] ^ (np.arange(31, dtype=np.uint16)[None, :] % 2 * 0x8000)
        elif fill == "random":
            blk[:, 1:] = rng.integers(0, 65536, size=(65536, 31), dtype=np.uint16)
        _check_dim0(blk.reshape(512, 4096), mode_name, mode, device)


@pytest.mark.parametrize("mode_name,mode", MODES)
def test_every_bf16_value_dim1(device, mode_name, mode):
    """Same sweep through the column-wise kernel: blocks run down 32 rows."""
    rng = np.random.default_rng(1)
    blk = rng.integers(0, 65536, size=(65536, 32), dtype=np.uint16)
    blk[:, 0] = np.arange(65536, dtype=np.uint16)
    # lay the 65536 blocks out as columns: x[32*g + k, c] = blk[g*512 + c, k]
    x = np.ascontiguousarray(blk.reshape(128, 512, 32).transpose(0, 2, 1)).reshape(128 * 32, 512)
    _check_dim1(x, mode_name, mode, device)
    _check_fused(x, mode_name, mode, device)


@pytest.mark.parametrize("mode_name,mode", MODES)
@pytest.mark.parametrize("shape", [(32, 32), (64, 96), (96, 64), (160, 224), (128, 128),
                                   (256, 4096), (1024, 768), (416, 2048), (32, 14336)])
def test_shapes_with_outliers(device, mode_name, mode, shape):
    rng = np.random.default_rng(hash(shape) & 0xFFFF)
    bits = randn_bits(rng, shape, outliers=1e-3)
    _check_dim0(bits, mode_name, mode, device)
    _check_dim1(bits, mode_name, mode, device)
    _check_fused(bits, mode_name, mode, device)


def test_dim1_equals_dim0_of_transpose(device):
    rng = np.random.default_rng(7)
    bits = randn_bits(rng, (512, 1024), outliers=1e-3)
    x = bf16_from_bits(bits, device)
    a = ops.to_mx_dim1(x, "rceil")
    b = ops.to_mx_dim0(x.t().contiguous(), "rceil")
    assert torch.equal(a.codes, b.codes) and torch.equal(a.scales, b.scales)


def test_strided_input_rows(device):
    rng = np.random.default_rng(8)
    bits = randn_bits(rng, (128, 512))
    x = bf16_from_bits(bits, device)
    view = x[:, :256]  # row stride 512, 256 columns
    got = ops.to_mx_dim0(view, "floor")
    codes, scales = mo.cast_dim0(bits[:, :256], mo.FLOOR)
    assert np.array_equal(u8(got.codes), codes) and np.array_equal(u8(got.scales), scales)
    got1 = ops.to_mx_dim1(view, "floor")
    codes1, scales1 = mo.cast_dim1(bits[:, :256], mo.FLOOR)
    assert np.array_equal(u8(got1.codes), codes1) and np.array_equal(u8(got1.scales), scales1)


def test_scale_layout_round_trip(device):
    rng = np.random.default_rng(9)
    for rows, nblk in [(64, 4), (100, 7), (256, 128), (4096, 448), (33, 1)]:
        s = rng.integers(0, 256, size=(rows, nblk), dtype=np.uint8)
        t = torch.from_numpy(s).to(device)
        laid = ops.scale_layout(t)
        assert np.array_equal(u8(laid), mo.scale_layout(s).reshape(-1))
        back = ops.scale_unlayout(laid, rows, nblk)
        assert np.array_equal(u8(back), s)


def test_empty_and_errors(device):
    x = torch.empty((0, 64), dtype=torch.bfloat16, device=device)
    out = ops.to_mx_dim0(x)
    assert out.codes.shape == (0, 64)
    with pytest.raises(ValueError):
        ops.to_mx_dim0(torch.zeros((4, 48), dtype=torch.bfloat16, device=device))
    with pytest.raises(ValueError):
        ops.to_mx_dim1(torch.zeros((48, 64), dtype=torch.bfloat16, device=device))
    with pytest.raises(TypeError):
        ops.to_mx_dim0(torch.zeros((4, 64), dtype=torch.float32, device=device))
    with pytest.raises(Exception):
        ops.to_mx_dim0(torch.zeros((4, 64), dtype=torch.bfloat16))  # CPU tensor: no fallback


def test_full_size_properties(device):
    """Benchmark-size tensor: properties that need no CPU oracle pass over the whole tensor."""
    torch.manual_seed(0)
    x = torch.randn((16384, 4096), device=device, dtype=torch.bfloat16)
    r, c = ops.to_mx_dim0_dim1(x, "floor")
    r2 = ops.to_mx_dim0(x, "floor")
    c2 = ops.to_mx_dim1(x, "floor")
    assert torch.equal(r.codes, r2.codes) and torch.equal(r.scales, r2.scales)
    assert torch.equal(c.codes, c2.codes) and torch.equal(c.scales, c2.scales)
    # idempotence under transpose
    ct = ops.to_mx_dim0(x.t().contiguous(), "floor")
    assert torch.equal(ct.codes, c.codes) and torch.equal(ct.scales, c.scales)
    # the oracle on a slice
    sl = bits_of(x[4096:4096 + 64])
    codes, scales = mo.cast_dim0(sl, mo.FLOOR)
    assert np.array_equal(u8(r.codes[4096:4096 + 64]), codes)
    assert np.array_equal(u8(r.scales[4096:4096 + 64]), scales)


def _check_gate(g_bits, a_bits, b_bits):
    """g equals the oracle's silu(a) * b, or, at a few elements in ten thousand, the product formed
    from a bf16 neighbour of silu(a) (a float32 silu rounding to the other side of a boundary)."""
    s = mo.silu_bf16(a_bits)
    exact = mo.mul_bf16(s, b_bits)
    nan = lambda x: (x & 0x7FFF) > 0x7F80
    same = (g_bits == exact) | (nan(g_bits) & nan(exact))
    movable = ((s & 0x7FFF) > 0) & ((s & 0x7FFF) < 0x7F7F)
    near = np.zeros_like(same)
    for step in (-1, 1):
        alt = mo.mul_bf16(np.where(movable, s.astype(np.int32) + step, s).astype(np.uint16), b_bits)
        near |= g_bits == alt
    assert (same | near).all(), int((~(same | near)).sum())
    assert (~same).mean() <= 2e-3, float((~same).mean())


@pytest.mark.parametrize("mode_name,mode", MODES)
@pytest.mark.parametrize("shape", [(32, 32), (160, 224), (256, 384), (1024, 768)])
def test_swiglu_fused_cast(device, mode_name, mode, shape):
    """g = silu(a) * b fused in front of both casts: g within one bf16 ulp of the oracle at a few
    elements in ten thousand and equal elsewhere; codes and scales exact for the g formed."""
    rng = np.random.default_rng(shape[0] * 13 + shape[1])
    a_bits = randn_bits(rng, shape, std=2.0, outliers=1e-3)
    b_bits = randn_bits(rng, shape, std=1.0)
    a, b = bf16_from_bits(a_bits, device), bf16_from_bits(b_bits, device)
    for order in (ops.MX_SCALES_ROWMAJOR, ops.MX_SCALES_MFMA):
        q0, q1, g = ops.swiglu_to_mx_dim0_dim1(a, b, mode_name, order, want_g=True)
        g_bits = bits_of(g)
        _check_gate(g_bits, a_bits, b_bits)
        c0, s0 = mo.cast_dim0(g_bits, mode)
        c1, s1 = mo.cast_dim1(g_bits, mode)
        if order == ops.MX_SCALES_MFMA:
            s0, s1 = mo.scale_layout(s0), mo.scale_layout(s1)
        assert np.array_equal(u8(q0.codes), c0) and np.array_equal(u8(q0.scales).reshape(-1), s0.reshape(-1))
        assert np.array_equal(u8(q1.codes), c1) and np.array_equal(u8(q1.scales).reshape(-1), s1.reshape(-1))
        # without the optional output the casts are the same
        p0, p1, none = ops.swiglu_to_mx_dim0_dim1(a, b, mode_name, order)
        assert none is None and torch.equal(p0.codes, q0.codes) and torch.equal(p1.scales, q1.scales)


def test_swiglu_fused_cast_special_values(device):
    """Zeros, large magnitudes, infinities and NaN go through the gate like the two tensor ops."""
    vals = np.array([0.0, -0.0, 1.0, -1.0, 30.0, -30.0, 88.0, -88.0, 100.0, -100.0, 1e30, -1e30,
                     np.inf, -np.inf, np.nan, 1e-30], dtype=np.float32)
    a = np.tile(vals, (32, 2))
    b = np.tile(vals[::-1].copy(), (32, 2))
    a_bits, b_bits = mo.f32_to_bf16_bits(a), mo.f32_to_bf16_bits(b)
    _, _, g = ops.swiglu_to_mx_dim0_dim1(bf16_from_bits(a_bits, device), bf16_from_bits(b_bits, device), "rceil", ops.MX_SCALES_ROWMAJOR, want_g=True)
    _check_gate(bits_of(g), a_bits, b_bits)


def test_swiglu_gate_every_bf16_input(device):
    """Every bf16 bit pattern as the gate input (denormals, the range where exp(-a) nears and
    passes float32's maximum, infinities, NaNs), against seeded multipliers: within the oracle's
    bound, and bit-identical to the two bf16 tensor ops run on the GPU by torch."""
    a_bits = np.arange(65536, dtype=np.uint16).reshape(256, 256)
    b_bits = randn_bits(np.random.default_rng(77), (256, 256), std=1.0)
    a, b = bf16_from_bits(a_bits, device), bf16_from_bits(b_bits, device)
    _, _, g = ops.swiglu_to_mx_dim0_dim1(a, b, "floor", ops.MX_SCALES_MFMA, want_g=True)
    _check_gate(bits_of(g), a_bits, b_bits)
    want = torch.nn.functional.silu(a) * b
    both_nan = torch.isnan(g) & torch.isnan(want)
    assert torch.equal(g.view(torch.int16)[~both_nan], want.view(torch.int16)[~both_nan])


def _equal_or_nan(got, want):
    both_nan = torch.isnan(got) & torch.isnan(want)
    return torch.equal(got.view(torch.int16)[~both_nan], want.view(torch.int16)[~both_nan])


@pytest.mark.parametrize("mode_name,mode", MODES)
@pytest.mark.parametrize("shape", [(32, 32), (160, 224), (256, 384), (1024, 768)])
def test_swiglu_backward_fused_cast(device, mode_name, mode, shape):
    """Gate backward fused in front of four casts: gradients within the oracle's bound (db exact,
    da equal or the neighbouring bf16 value at a few elements in ten thousand) and bit-identical
    to torch's GPU autograd of the two bf16 ops; codes and scales exact for those gradients."""
    rng = np.random.default_rng(shape[0] * 7 + shape[1])
    a_bits = randn_bits(rng, shape, std=2.0, outliers=1e-3)
    b_bits = randn_bits(rng, shape, std=1.0)
    dg_bits = randn_bits(rng, shape, std=0.5, outliers=1e-3)
    a, b, dg = (bf16_from_bits(x, device) for x in (a_bits, b_bits, dg_bits))
    ta, tb = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
    (torch.nn.functional.silu(ta) * tb).backward(dg)
    da_o, db_o = mo.swiglu_backward_bf16(dg_bits, a_bits, b_bits)
    for order in (ops.MX_SCALES_ROWMAJOR, ops.MX_SCALES_MFMA):
        qa, qb, grads = ops.swiglu_bwd_to_mx_dim0_dim1(dg, a, b, mode_name, order, want_grads=True)
        assert _equal_or_nan(grads[0], ta.grad) and _equal_or_nan(grads[1], tb.grad)
        da_bits, db_bits = bits_of(grads[0]), bits_of(grads[1])
        nan = lambda x: (x & 0x7FFF) > 0x7F80
        assert ((db_bits == db_o) | (nan(db_bits) & nan(db_o))).all()
        off = (da_bits != da_o) & ~(nan(da_bits) & nan(da_o))
        assert off.mean() <= 2e-3
        assert (np.abs(da_bits[off].astype(np.int32) - da_o[off].astype(np.int32)) <= 1).all()
        for (q0, q1), bits in ((qa, da_bits), (qb, db_bits)):
            c0, s0 = mo.cast_dim0(bits, mode)
            c1, s1 = mo.cast_dim1(bits, mode)
            if order == ops.MX_SCALES_MFMA:
                s0, s1 = mo.scale_layout(s0), mo.scale_layout(s1)
            assert np.array_equal(u8(q0.codes), c0) and np.array_equal(u8(q0.scales).reshape(-1), s0.reshape(-1))
            assert np.array_equal(u8(q1.codes), c1) and np.array_equal(u8(q1.scales).reshape(-1), s1.reshape(-1))
        pa, pb, none = ops.swiglu_bwd_to_mx_dim0_dim1(dg, a, b, mode_name, order)
        assert none is None and torch.equal(pa[0].codes, qa[0].codes) and torch.equal(pb[1].codes, qb[1].codes)
        assert torch.equal(pa[1].scales, qa[1].scales) and torch.equal(pb[0].scales, qb[0].scales)


def test_swiglu_backward_every_bf16_gate_input(device):
    """Every bf16 bit pattern as the gate input, against torch's GPU autograd."""
    rng = np.random.default_rng(78)
    a = bf16_from_bits(np.arange(65536, dtype=np.uint16).reshape(256, 256), device)
    for std in (1.0, 30.0):
        b = bf16_from_bits(randn_bits(rng, (256, 256), std=std), device)
        dg = bf16_from_bits(randn_bits(rng, (256, 256), std=std), device)
        ta, tb = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
        (torch.nn.functional.silu(ta) * tb).backward(dg)
        _, _, grads = ops.swiglu_bwd_to_mx_dim0_dim1(dg, a, b, "rceil", ops.MX_SCALES_MFMA, want_grads=True)
        assert _equal_or_nan(grads[0], ta.grad) and _equal_or_nan(grads[1], tb.grad)


@pytest.mark.parametrize("mode_name,mode", MODES)
@pytest.mark.parametrize("src_rows,rows,cols", [(50, 64, 96), (300, 512, 256), (1000, 1184, 160)])
def test_cast_of_gathered_rows(device, mode_name, mode, src_rows, rows, cols):
    """Cast of x[row_index] with -1 (and out-of-range) slots as zero rows == cast of the tensor
    the gather would have formed; with and without the column-wise output."""
    rng = np.random.default_rng(rows + cols)
    bits = randn_bits(rng, (src_rows, cols), outliers=1e-3)
    idx = np.full(rows, -1, dtype=np.int64)
    slots = rng.permutation(rows)[:src_rows] if src_rows <= rows else rng.permutation(rows)
    idx[slots] = rng.permutation(src_rows)[:len(slots)]
    idx[rng.integers(0, rows)] = src_rows + 5  # outside the source: zeros as well
    valid = (idx >= 0) & (idx < src_rows)
    gathered = np.where(valid[:, None], bits[np.clip(idx, 0, src_rows - 1)], 0).astype(np.uint16)
    x = bf16_from_bits(bits, device)
    ti = torch.from_numpy(idx).to(device)
    for order in (ops.MX_SCALES_ROWMAJOR, ops.MX_SCALES_MFMA):
        q0, q1 = ops.to_mx_rows_gathered(x, ti, mode_name, order)
        c0, s0 = mo.cast_dim0(gathered, mode)
        c1, s1 = mo.cast_dim1(gathered, mode)
        if order == ops.MX_SCALES_MFMA:
            s0, s1 = mo.scale_layout(s0), mo.scale_layout(s1)
        assert np.array_equal(u8(q0.codes), c0) and np.array_equal(u8(q0.scales).reshape(-1), s0.reshape(-1))
        assert np.array_equal(u8(q1.codes), c1) and np.array_equal(u8(q1.scales).reshape(-1), s1.reshape(-1))
        r0, none = ops.to_mx_rows_gathered(x, ti, mode_name, order, want_cols=False)
        assert none is None and torch.equal(r0.codes, q0.codes) and torch.equal(r0.scales, q0.scales)


@pytest.mark.parametrize("mode_name,mode", MODES)
def test_cast_of_gathered_rows_with_scores(device, mode_name, mode):
    """The routing-score multiply in front of the experts folded into the gathered cast."""
    rng = np.random.default_rng(31)
    src_rows, rows, cols = 200, 672, 192
    bits = randn_bits(rng, (src_rows, cols), outliers=1e-3)
    idx = rng.integers(-1, src_rows, rows).astype(np.int64)
    scale = rng.random(rows).astype(np.float32) * 2
    gathered = mo.gather_rows(bits, idx, scale)
    q0, q1 = ops.to_mx_rows_gathered(bf16_from_bits(bits, device), torch.from_numpy(idx).to(device), mode_name,
                                     ops.MX_SCALES_MFMA, row_scale=torch.from_numpy(scale).to(device))
    c0, s0 = mo.cast_dim0(gathered, mode)
    c1, s1 = mo.cast_dim1(gathered, mode)
    assert np.array_equal(u8(q0.codes), c0) and np.array_equal(u8(q0.scales).reshape(-1), mo.scale_layout(s0).reshape(-1))
    assert np.array_equal(u8(q1.codes), c1) and np.array_equal(u8(q1.scales).reshape(-1), mo.scale_layout(s1).reshape(-1))


@pytest.mark.parametrize("tokens,k,cols", [(64, 1, 64), (300, 4, 256), (1000, 8, 2048)])
def test_moe_combine_and_row_dot(device, tokens, k, cols):
    """Weighted top-k combine bit-exact against the oracle's float32 sequential sum; score
    gradients (row dot products) to 1e-5 of the float64 oracle (float32 reduction)."""
    rng = np.random.default_rng(tokens + k)
    rows = tokens * k + 40
    y_bits = randn_bits(rng, (rows, cols))
    pos = rng.permutation(rows)[: tokens * k].astype(np.int64).reshape(tokens, k)
    pos[rng.integers(0, tokens), rng.integers(0, k)] = -1
    pos[rng.integers(0, tokens), rng.integers(0, k)] = rows + 3
    w = rng.random((tokens, k)).astype(np.float32)
    y = bf16_from_bits(y_bits, device)
    tp = torch.from_numpy(pos).to(device)
    got = ops.moe_combine(y, tp, torch.from_numpy(w).to(device))
    assert np.array_equal(bits_of(got), mo.moe_combine(y_bits, pos, w))
    got = ops.moe_combine(y, tp)
    assert np.array_equal(bits_of(got), mo.moe_combine(y_bits, pos, None))
    # two partial matrices merged by a bf16 addition on the way in
    y2_bits = randn_bits(rng, (rows, cols))
    y2 = bf16_from_bits(y2_bits, device)
    merged = mo.add_bf16(y_bits, y2_bits)
    got = ops.moe_combine(y, tp, torch.from_numpy(w).to(device), y2)
    assert np.array_equal(bits_of(got), mo.moe_combine(merged, pos, w))
    x_bits = randn_bits(rng, (tokens, cols))
    ib = (np.arange(tokens * k) // k).astype(np.int64)
    d = ops.moe_row_dot(y, tp.view(-1), bf16_from_bits(x_bits, device), torch.from_numpy(ib).to(device))
    ref = mo.moe_row_dot(y_bits, pos.reshape(-1), x_bits, ib)
    assert np.allclose(d.cpu().numpy().astype(np.float64), ref, rtol=1e-5, atol=1e-5 * np.sqrt(cols))
    d = ops.moe_row_dot(y, tp.view(-1), bf16_from_bits(x_bits, device), torch.from_numpy(ib).to(device), y2)
    ref = mo.moe_row_dot(merged, pos.reshape(-1), x_bits, ib)
    assert np.allclose(d.cpu().numpy().astype(np.float64), ref, rtol=1e-5, atol=1e-5 * np.sqrt(cols))


@pytest.mark.parametrize("mode_name,mode", MODES)
def test_dequant_is_exact(device, mode_name, mode):
    """codes x 2^(scale - 127) back to bf16: equal to the oracle's dequantization bit for bit, in
    both scale orders, including all-zero blocks, a NaN block and the smallest scales."""
    rng = np.random.default_rng(8)
    bits = randn_bits(rng, (192, 160), outliers=1e-2)
    bits[3, 32:64] = 0
    bits[5, 70] = 0x7FC0
    bits[7, :32] = mo.f32_to_bf16_bits((rng.standard_normal(32) * 1e-38).astype(np.float32))
    x = bf16_from_bits(bits, device)
    for order in (ops.MX_SCALES_ROWMAJOR, ops.MX_SCALES_MFMA):
        q = ops.to_mx_dim0(x, mode_name, order)
        got = bits_of(ops.mx_dequant(q))
        codes, scales = mo.cast_dim0(bits, mode)
        want = mo.f32_to_bf16_bits(mo.dequant(codes, scales))
        nan = lambda v: (v & 0x7FFF) > 0x7F80
        assert (nan(got) == nan(want)).all() and np.array_equal(got[~nan(want)], want[~nan(want)])


def test_fused_casts_at_benchmark_sizes_equal_separate_kernels(device):
    """At the sizes the benchmark runs (16384 x 14336 activations; 139264 padded rows of 2048 for
    the MoE config) the gate-fused and gathered casts equal the plain cast of the tensor the
    separate ops would have formed, byte for byte."""
    torch.manual_seed(3)
    M, H = 16384, 14336
    a = (torch.randn(M, H, device=device) * 2).to(torch.bfloat16)
    b = torch.randn(M, H, device=device).to(torch.bfloat16)
    L = ops.MX_SCALES_MFMA
    q0, q1, _ = ops.swiglu_to_mx_dim0_dim1(a, b, "rceil", L)
    g = torch.nn.functional.silu(a) * b
    r0, r1 = ops.to_mx_dim0_dim1(g, "rceil", L)
    for got, want in ((q0, r0), (q1, r1)):
        assert torch.equal(got.codes, want.codes) and torch.equal(got.scales, want.scales)
    del q0, q1, r0, r1, g
    dg = (torch.randn(M, H, device=device) * 1e-3).to(torch.bfloat16)
    ta, tb = a.clone().requires_grad_(True), b.clone().requires_grad_(True)
    (torch.nn.functional.silu(ta) * tb).backward(dg)
    (da0, da1), (db0, db1), _ = ops.swiglu_bwd_to_mx_dim0_dim1(dg, a, b, "rceil", L)
    for (got0, got1), grad in (((da0, da1), ta.grad), ((db0, db1), tb.grad)):
        w0, w1 = ops.to_mx_dim0_dim1(grad, "rceil", L)
        assert torch.equal(got0.codes, w0.codes) and torch.equal(got0.scales, w0.scales)
        assert torch.equal(got1.codes, w1.codes) and torch.equal(got1.scales, w1.scales)
    del a, b, dg, ta, tb, da0, da1, db0, db1, w0, w1
    torch.cuda.empty_cache()
    T, k, D, rows = 16384, 8, 2048, 139264
    x = torch.randn(T, D, device=device).to(torch.bfloat16)
    idx = torch.full((rows,), -1, dtype=torch.int64, device=device)
    slots = torch.randperm(rows, device=device)[: T * k]
    idx[slots] = torch.randint(0, T, (T * k,), device=device)
    score = torch.rand(rows, device=device)
    q0, q1 = ops.to_mx_rows_gathered(x, idx, "rceil", L, row_scale=score)
    gathered = torch.cat((x, x.new_zeros((1, D))))[idx]
    gathered = (gathered.float() * score[:, None]).to(torch.bfloat16)
    r0, r1 = ops.to_mx_dim0_dim1(gathered, "rceil", L)
    for got, want in ((q0, r0), (q1, r1)):
        assert torch.equal(got.codes, want.codes) and torch.equal(got.scales, want.scales)


@pytest.mark.parametrize("mode_name,mode", MODES)
@pytest.mark.parametrize("shape", [(32, 64), (160, 224), (512, 4096)])
def test_rms_norm_fused_cast(device, mode_name, mode, shape):
    """RMSNorm in front of both casts: rstd to 1e-6 of the float64 oracle; y equal to the oracle's
    or the neighbouring bf16 value (float32 reduction), and likewise against torch's GPU
    rms_norm; codes and scales exact for the y that was formed."""
    rng = np.random.default_rng(shape[0] + shape[1])
    x_bits = randn_bits(rng, shape, std=2.0, outliers=1e-3)
    w_bits = mo.f32_to_bf16_bits((1 + 0.2 * rng.standard_normal(shape[1])).astype(np.float32))
    x, w = bf16_from_bits(x_bits, device), bf16_from_bits(w_bits, device)
    y_o, rstd_o = mo.rms_norm_bf16(x_bits, w_bits, 1e-5)
    y_t = bits_of(torch.nn.functional.rms_norm(x, (shape[1],), w, 1e-5))
    for order in (ops.MX_SCALES_ROWMAJOR, ops.MX_SCALES_MFMA):
        q0, q1, rstd, y = ops.rms_norm_to_mx(x, w, 1e-5, mode_name, order, want_y=True)
        assert np.allclose(rstd.cpu().numpy(), rstd_o, rtol=2e-6)
        y_bits = bits_of(y)
        for ref in (y_o, y_t):
            off = y_bits != ref
            assert off.mean() < 0.02 and (np.abs(y_bits[off].astype(np.int32) - ref[off].astype(np.int32)) <= 1).all()
        c0, s0 = mo.cast_dim0(y_bits, mode)
        c1, s1 = mo.cast_dim1(y_bits, mode)
        if order == ops.MX_SCALES_MFMA:
            s0, s1 = mo.scale_layout(s0), mo.scale_layout(s1)
        assert np.array_equal(u8(q0.codes), c0) and np.array_equal(u8(q0.scales).reshape(-1), s0.reshape(-1))
        assert np.array_equal(u8(q1.codes), c1) and np.array_equal(u8(q1.scales).reshape(-1), s1.reshape(-1))
        p0, p1, _, none = ops.rms_norm_to_mx(x, w, 1e-5, mode_name, order)
        assert none is None and torch.equal(p0.codes, q0.codes) and torch.equal(p1.scales, q1.scales)


@pytest.mark.parametrize("R,C,pad", [(128, 256, 128), (4096, 4096, 128), (96, 160, 16), (1024, 14336, 384)])
def test_fused_cast_with_row_pitches_writes_the_same_codes(device, R, C, pad):
    """Codes whose rows lie `pad` bytes further apart than they are long: every row equals the
    dense cast's, the bytes between the rows are left alone, scales are unchanged."""
    torch.manual_seed(R + C)
    x = torch.randn(R, C, device=device, dtype=torch.bfloat16)
    x[3, 5] = 300.0
    for mode in ("floor", "rceil"):
        want0, want1 = ops.to_mx_dim0_dim1(x, mode, ops.MX_SCALES_MFMA)
        got0, got1 = ops.to_mx_dim0_dim1(x, mode, ops.MX_SCALES_MFMA, pitch_pad=pad)
        assert got0.codes.stride(0) == C + pad and got1.codes.stride(0) == R + pad
        assert torch.equal(got0.codes, want0.codes) and torch.equal(got1.codes, want1.codes)
        assert torch.equal(got0.scales, want0.scales) and torch.equal(got1.scales, want1.scales)
    # between the rows: untouched
    lib = _lib.load()
    base0 = torch.full((R, C + pad), 0xAB, dtype=torch.uint8, device=device)
    base1 = torch.full((C, R + pad), 0xCD, dtype=torch.uint8, device=device)
    s0 = torch.empty_like(want0.scales)
    s1 = torch.empty_like(want1.scales)
    with torch.cuda.device(device):
        st = lib.mx_cast_dim0_dim1_ld(ops._ptr(x), R, C, x.stride(0), ops._ptr(base0), C + pad, ops._ptr(s0),
                                      ops._ptr(base1), R + pad, ops._ptr(s1), 1, ops.MX_SCALES_MFMA, ops._stream(x))
    assert st == 0
    assert bool((base0[:, C:] == 0xAB).all()) and bool((base1[:, R:] == 0xCD).all())
    assert torch.equal(base0[:, :C], want0.codes) and torch.equal(base1[:, :R], want1.codes)


@pytest.mark.parametrize("R,C,pad", [(160, 224, 128), (1024, 768, 128), (96, 160, 16)])
def test_gate_and_norm_casts_with_row_pitches_write_the_same_codes(device, R, C, pad):
    """The SwiGLU forward and backward casts and the RMSNorm cast with a row pitch: codes, scales
    and optional bf16 outputs equal those of the dense forms; through the C ABI the bytes between
    the rows (and between the two halves of the backward cast) are left alone."""
    torch.manual_seed(R * 3 + C)
    a, b, dg = (torch.randn(R, C, device=device, dtype=torch.bfloat16) * s for s in (2.0, 1.0, 0.5))
    w = (1 + 0.2 * torch.randn(C, device=device)).to(torch.bfloat16)
    L = ops.MX_SCALES_MFMA
    eq = lambda p, q: (p.codes.stride(0) == q.codes.shape[1] + pad and torch.equal(p.codes, q.codes)
                       and torch.equal(p.scales, q.scales))
    for mode in ("floor", "rceil"):
        d0, d1, dgate = ops.swiglu_to_mx_dim0_dim1(a, b, mode, L, want_g=True)
        p0, p1, pgate = ops.swiglu_to_mx_dim0_dim1(a, b, mode, L, want_g=True, pitch_pad=pad)
        assert eq(p0, d0) and eq(p1, d1) and torch.equal(pgate, dgate)
        (da0, da1), (db0, db1), dgr = ops.swiglu_bwd_to_mx_dim0_dim1(dg, a, b, mode, L, want_grads=True)
        (pa0, pa1), (pb0, pb1), pgr = ops.swiglu_bwd_to_mx_dim0_dim1(dg, a, b, mode, L, want_grads=True, pitch_pad=pad)
        assert eq(pa0, da0) and eq(pa1, da1) and eq(pb0, db0) and eq(pb1, db1) and torch.equal(pgr, dgr)
        n0, n1, rstd, y = ops.rms_norm_to_mx(a, w, 1e-5, mode, L, want_y=True)
        q0, q1, prstd, py = ops.rms_norm_to_mx(a, w, 1e-5, mode, L, want_y=True, pitch_pad=pad)
        assert eq(q0, n0) and eq(q1, n1) and torch.equal(prstd, rstd) and torch.equal(py, y)
    # the backward cast through the C ABI into buffers filled with a marker
    lib = _lib.load()
    (da0, da1), (db0, db1), _ = ops.swiglu_bwd_to_mx_dim0_dim1(dg, a, b, "rceil", L)
    c = torch.full((2, R, C + pad), 0xAB, dtype=torch.uint8, device=device)
    ct = torch.full((2, C, R + pad), 0xCD, dtype=torch.uint8, device=device)
    s = torch.empty(2 * da0.scales.numel(), dtype=torch.uint8, device=device)
    st_ = torch.empty(2 * da1.scales.numel(), dtype=torch.uint8, device=device)
    with torch.cuda.device(device):
        rc = lib.mx_swiglu_bwd_cast_dim0_dim1_ld(ops._ptr(dg), ops._ptr(a), ops._ptr(b), R, C, C, C, C, ops._ptr(c), C + pad,
                                                 ops._ptr(s), ops._ptr(ct), R + pad, ops._ptr(st_), None, 1, L,
                                                 ops._stream(a))
    assert rc == 0
    assert bool((c[:, :, C:] == 0xAB).all()) and bool((ct[:, :, R:] == 0xCD).all())
    assert torch.equal(c[0, :, :C], da0.codes) and torch.equal(c[1, :, :C], db0.codes)
    assert torch.equal(ct[0, :, :R], da1.codes) and torch.equal(ct[1, :, :R], db1.codes)
    assert torch.equal(s[:da0.scales.numel()], da0.scales.reshape(-1)) and torch.equal(st_[da1.scales.numel():], db1.scales.reshape(-1))
    # pitches that are too small or not multiples of 16 are refused
    with torch.cuda.device(device):
        assert lib.mx_swiglu_cast_dim0_dim1_ld(ops._ptr(a), ops._ptr(b), R, C, C, C, ops._ptr(c), C - 16, ops._ptr(s),
                                               ops._ptr(ct), R + pad, ops._ptr(st_), None, 1, L, ops._stream(a)) != 0
        assert lib.mx_swiglu_cast_dim0_dim1_ld(ops._ptr(a), ops._ptr(b), R, C, C, C, ops._ptr(c), C + 8, ops._ptr(s),
                                               ops._ptr(ct), R + pad, ops._ptr(st_), None, 1, L, ops._stream(a)) != 0
