"""Pins the CPU oracle to things it did not produce itself: torch's CPU float8/bfloat16 casts
(library routines), hand-computed known answers (tests/golden/known_answers.json), closed forms
evaluated in exact arithmetic, brute force, an independent C restatement, and the worked
example of the reference's permute-index docstring."""
import json
import math
from fractions import Fraction
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import mx_oracle as mo

GOLDEN = Path(__file__).parent / "golden"
ALL_BF16 = np.arange(65536, dtype=np.uint16)


# ------------------------------------------------------------------ element formats
def test_e4m3_decode_table_vs_torch():
    codes = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    got = mo.e4m3_decode(codes)
    assert np.array_equal(np.isnan(ref), np.isnan(got))
    assert np.array_equal(ref[~np.isnan(ref)], got[~np.isnan(got)])
    assert np.signbit(got[0x80]) and got[0x80] == 0 and got[0x7E] == 448 and got[0x01] == 2.0 ** -9


def test_e4m3_encode_vs_torch_all_bf16_and_random_f32():
    f = mo.bf16_bits_to_f32(ALL_BF16)
    rng = np.random.default_rng(0)
    extra = (rng.standard_normal(200000) * np.exp(rng.uniform(-12, 8, 200000))).astype(np.float32)
    ties = np.concatenate([(mo.e4m3_decode(np.arange(0x7E, dtype=np.uint8)) + mo.e4m3_decode(np.arange(1, 0x7F, dtype=np.uint8))) / 2])
    vals = np.concatenate([f, extra, ties.astype(np.float32), -ties.astype(np.float32)])
    finite = ~np.isnan(vals)
    ref = torch.clamp(torch.from_numpy(vals[finite].copy()), -448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(mo.e4m3_encode(vals[finite]), ref)
    nan_codes = mo.e4m3_encode(vals[~finite])
    assert set(nan_codes.tolist()) <= {0x7F, 0xFF}


def test_encode_decode_round_trip_all_codes():
    codes = np.array([c for c in range(256) if c & 0x7F != 0x7F], dtype=np.uint8)
    assert np.array_equal(mo.e4m3_encode(mo.e4m3_decode(codes)), codes)


def test_bf16_conversions_vs_torch():
    f = mo.bf16_bits_to_f32(ALL_BF16)
    ref = torch.from_numpy(ALL_BF16.view(np.int16)).view(torch.bfloat16).float().numpy()
    assert np.array_equal(f.view(np.uint32), ref.view(np.uint32))
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(300000) * np.exp(rng.uniform(-30, 30, 300000))).astype(np.float32)
    ref = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(mo.f32_to_bf16_bits(x), ref)


def test_rms_norm_vs_torch_cpu():
    """Oracle RMSNorm against torch's CPU op on bf16 tensors: equal except where float32
    arithmetic lands on the neighbouring bf16 value."""
    rng = np.random.default_rng(12)
    x = mo.f32_to_bf16_bits((rng.standard_normal((64, 512)) * 3).astype(np.float32))
    w = mo.f32_to_bf16_bits((1 + 0.1 * rng.standard_normal(512)).astype(np.float32))
    t = lambda bits: torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    ref = torch.nn.functional.rms_norm(t(x), (512,), t(w), 1e-5).view(torch.int16).numpy().view(np.uint16)
    got, rstd = mo.rms_norm_bf16(x, w, 1e-5)
    off = got != ref
    assert off.mean() < 0.02
    assert (np.abs(got[off].astype(np.int32) - ref[off].astype(np.int32)) <= 1).all()
    xf = mo.bf16_bits_to_f32(x).astype(np.float64)
    assert np.allclose(rstd, 1 / np.sqrt((xf ** 2).mean(1) + 1e-5))


def test_swiglu_vs_torch_bf16_ops_every_gate_input():
    """silu over every bf16 bit pattern, and the gate product on a random pairing, against
    torch's CPU bf16 tensor ops (the ops feed_forward.py:61-62 runs)."""
    t = lambda bits: torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    b = lambda x: x.view(torch.int16).numpy().view(np.uint16)
    nan = lambda x: (x & 0x7FFF) > 0x7F80
    s_ref = b(torch.nn.functional.silu(t(ALL_BF16)))
    s = mo.silu_bf16(ALL_BF16)
    assert np.array_equal(np.where(nan(s), 0x7FC0, s), np.where(nan(s_ref), 0x7FC0, s_ref))
    other = np.random.default_rng(5).permutation(ALL_BF16)
    g_ref = b(torch.nn.functional.silu(t(ALL_BF16)) * t(other))
    g = mo.swiglu_bf16(ALL_BF16, other)
    assert np.array_equal(np.where(nan(g), 0x7FC0, g), np.where(nan(g_ref), 0x7FC0, g_ref))


def test_swiglu_backward_vs_torch_autograd_and_central_difference():
    """Gate gradients against torch's CPU bf16 autograd over every bf16 gate input (db exact; da
    equal except where a float32 evaluation rounds to the neighbouring bf16 value), and the
    float64 derivative inside against a central difference."""
    t = lambda bits: torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    b = lambda x: x.view(torch.int16).numpy().view(np.uint16)
    nan = lambda x: (x & 0x7FFF) > 0x7F80
    rng = np.random.default_rng(3)
    dg = mo.f32_to_bf16_bits(rng.standard_normal(65536).astype(np.float32))
    h3 = mo.f32_to_bf16_bits(rng.standard_normal(65536).astype(np.float32))
    da, db = mo.swiglu_backward_bf16(dg, ALL_BF16, h3)
    ta, tb = t(ALL_BF16).clone().requires_grad_(True), t(h3).clone().requires_grad_(True)
    (torch.nn.functional.silu(ta) * tb).backward(t(dg))
    ra, rb = b(ta.grad), b(tb.grad)
    assert not ((db != rb) & ~(nan(db) & nan(rb))).any()
    off = (da != ra) & ~(nan(da) & nan(ra))
    assert off.sum() <= 4
    assert (np.abs(da[off].astype(np.int32) - ra[off].astype(np.int32)) <= 1).all()
    # d/da [a * sigmoid(a)] = s * (1 + a * (1 - s))
    x = np.linspace(-20, 20, 4001)
    silu = lambda v: v / (1 + np.exp(-v))
    s = 1 / (1 + np.exp(-x))
    assert np.allclose(s * (1 + x * (1 - s)), (silu(x + 1e-6) - silu(x - 1e-6)) / 2e-6, atol=1e-8)


def test_moe_gather_and_combine_vs_torch_cpu_ops():
    """gather_rows against torch indexing + the float32 score multiply; moe_combine against the
    reference's un-sort scatter + float bmm / sum (moe.py:519-555) run with torch on the CPU and
    against an exact float64 sum."""
    rng = np.random.default_rng(9)
    T, k, D = 96, 4, 64
    t = lambda bits: torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    b = lambda x: x.contiguous().view(torch.int16).numpy().view(np.uint16)
    x = mo.f32_to_bf16_bits(rng.standard_normal((T, D)).astype(np.float32))
    scores = rng.random((T, k)).astype(np.float32)
    order = rng.permutation(T * k)  # token_indices_experts_sorted
    # dispatch: routed_input = (x[order // k].float() * scores_sorted).to(bf16)
    want = (t(x)[torch.from_numpy(order // k)].float() * torch.from_numpy(scores.reshape(-1)[order])[:, None]).to(torch.bfloat16)
    got = mo.gather_rows(x, order // k, scores.reshape(-1)[order])
    assert np.array_equal(got, b(want))
    idx = np.array([3, -1, T + 2, 0])
    assert np.array_equal(mo.gather_rows(x, idx)[[1, 2]], np.zeros((2, D), np.uint16))
    assert np.array_equal(mo.gather_rows(x, idx)[[0, 3]], x[[3, 0]])
    # combine: y rows in sorted order; unsorted[order] = y; out = bmm(scores, unsorted.float())
    y = mo.f32_to_bf16_bits(rng.standard_normal((T * k, D)).astype(np.float32))
    pos = np.empty(T * k, dtype=np.int64)
    pos[order] = np.arange(T * k)
    pos = pos.reshape(T, k)
    unsorted = torch.zeros((T * k, D), dtype=torch.bfloat16)
    unsorted[torch.from_numpy(order)] = t(y)
    unsorted = unsorted.reshape(T, k, D)
    exact = lambda w: np.einsum("tk,tkd->td", w.astype(np.float64), mo.bf16_bits_to_f32(b(unsorted)).astype(np.float64))
    near = lambda got, ex: np.abs(mo.bf16_bits_to_f32(got).astype(np.float64) - ex) <= np.abs(ex) * 2.0 ** -8 + 1e-30
    for w in (scores, None):
        got = mo.moe_combine(y, pos, w)
        ref = (torch.bmm(torch.from_numpy(scores).reshape(T, 1, k), unsorted.float()).to(torch.bfloat16).squeeze(1)
               if w is not None else unsorted.sum(dim=1))
        differ = got != b(ref)
        assert differ.mean() < 0.02          # only accumulation-order effects
        assert near(got, exact(w if w is not None else np.ones((T, k), np.float32))).all()
    d = mo.moe_row_dot(y, pos.reshape(-1), x, np.arange(T * k) // k)
    ref = (unsorted.float() * t(x).float()[:, None, :]).sum(-1).numpy().reshape(-1)
    assert np.allclose(d, ref, rtol=1e-4, atol=1e-5)


# ------------------------------------------------------------------ scales
def _normal_finite():
    a = ALL_BF16[(ALL_BF16 >= 0x0080) & (ALL_BF16 < 0x7F80)]
    return a, mo.bf16_bits_to_f32(a).astype(np.float64)


def test_floor_scale_closed_form_every_normal_amax():
    bits, val = _normal_finite()
    expect = np.array([min(max(math.frexp(v)[1] - 1 - 8, -127), 127) + 127 for v in val])
    assert np.array_equal(mo.scale_from_amax_bits(bits, mo.FLOOR), expect)


def test_rceil_scale_closed_form_every_normal_amax():
    """ceil(log2(amax / 448)) in exact rational arithmetic: smallest s with amax <= 448 * 2^s."""
    bits, val = _normal_finite()
    got = mo.scale_from_amax_bits(bits, mo.RCEIL).astype(int) - 127
    for b, v, s in zip(bits[::7], val[::7], got[::7]):
        q = Fraction(v) / 448
        s_true = math.ceil(math.log2(q)) if q.numerator != 1 and q.denominator != 1 else None
        # exact: 2^(s-1) < q <= 2^s
        lo = Fraction(2) ** (int(s) - 1)
        hi = Fraction(2) ** int(s)
        if -127 < s < 127:
            assert lo < q <= hi, (hex(b), v, s, s_true)


def test_scale_byte_monotone_in_amax():
    bits = ALL_BF16[ALL_BF16 <= 0x7F80]
    for mode in (mo.FLOOR, mo.RCEIL):
        s = mo.scale_from_amax_bits(bits, mode).astype(int)
        assert np.all(np.diff(s) >= 0)
        assert s[0] == 0 and mo.scale_from_amax_bits(np.array([0x7FC0], np.uint16), mode)[0] == 255


def test_known_answers():
    data = json.loads((GOLDEN / "known_answers.json").read_text())
    for case in data["cases"]:
        blk = np.zeros((1, 32), np.float32)
        blk[0, 0] = case["value"]
        bits = mo.f32_to_bf16_bits(blk)
        for name, mode in (("floor", mo.FLOOR), ("rceil", mo.RCEIL)):
            codes, scales = mo.cast_dim0(bits, mode)
            assert [int(scales[0, 0]), codes[0, 0]] == [case[name][0], int(case[name][1], 16)], (case, name)
            assert np.all(codes[0, 1:] == 0)
            cc, cs = co.cast_dim0(bits, mode)
            assert np.array_equal(cc, codes) and np.array_equal(cs, scales)
    for nb in data["neighbours"]:
        blk = np.zeros((1, 32), np.float32)
        blk[0, : len(nb["block"])] = nb["block"]
        codes, scales = mo.cast_dim0(mo.f32_to_bf16_bits(blk), mo.FLOOR if nb["mode"] == "floor" else mo.RCEIL)
        assert scales[0, 0] == nb["scale"]
        assert codes[0, : len(nb["codes"])].tolist() == [int(c, 16) for c in nb["codes"]]


# ------------------------------------------------------------------ cast invariants
def _cfg1_like(seed, shape):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(shape, dtype=np.float32)
    x = np.where(rng.random(shape) < 1e-3, x * 100, x)
    return mo.f32_to_bf16_bits(x)


@pytest.mark.parametrize("mode", [mo.FLOOR, mo.RCEIL])
def test_quantization_error_bound_and_saturation(mode):
    bits = _cfg1_like(2, (256, 1024))
    codes, scales = mo.cast_dim0(bits, mode)
    x = mo.bf16_bits_to_f32(bits).astype(np.float64).reshape(256, 32, 32)
    d = mo.dequant(codes, scales).astype(np.float64).reshape(256, 32, 32)
    s = np.exp2(scales.astype(np.float64) - 127)[..., None]
    y = np.abs(x) / s                       # magnitude on the e4m3 grid
    ulp = np.where(y < 2.0 ** -6, 2.0 ** -9, np.exp2(np.floor(np.log2(np.maximum(y, 1e-300))) - 3))
    saturated = y > 448
    assert np.all(np.abs(x - d)[~saturated] <= (ulp * s / 2 + 1e-300)[~saturated])
    assert np.all(np.abs(d[saturated]) == (448 * np.broadcast_to(s, d.shape))[saturated])
    if mode == mo.RCEIL:
        assert not saturated.any()          # RCEIL never clips a finite in-range value
        assert np.all(y.max(axis=-1) > 224 - 1e-9)  # and uses the top binade: amax/2^s in (224, 448]
    else:
        assert np.all((y.max(axis=-1) >= 256) & (y.max(axis=-1) < 512))  # amax/2^s in [256, 512)
        assert saturated.any()              # mantissa > 1.75 does clip under FLOOR


def test_dim1_is_dim0_of_transpose_and_blocks_are_independent():
    bits = _cfg1_like(3, (128, 96))
    for mode in (mo.FLOOR, mo.RCEIL):
        c1, s1 = mo.cast_dim1(bits, mode)
        c0, s0 = mo.cast_dim0(np.ascontiguousarray(bits.T), mode)
        assert np.array_equal(c1, c0) and np.array_equal(s1, s0)
        # casting one block alone gives the same bytes as inside the matrix
        cb, sb = mo.cast_dim0(bits[5:6, 32:64], mode)
        call, sall = mo.cast_dim0(bits, mode)
        assert np.array_equal(cb[0], call[5, 32:64]) and sb[0, 0] == sall[5, 1]


def test_special_blocks():
    z = np.zeros((1, 32), np.uint16)
    z[0, 3] = 0x8000  # -0.0
    for mode in (mo.FLOOR, mo.RCEIL):
        c, s = mo.cast_dim0(z, mode)
        assert s[0, 0] == 0 and c[0, 3] == 0x80 and c[0].sum() == 0x80
    n = mo.f32_to_bf16_bits(np.array([[np.nan, 1.0, -2.0, np.inf] + [0.0] * 28], np.float32))
    c, s = mo.cast_dim0(n, mo.FLOOR)
    assert s[0, 0] == 255 and c[0, 0] in (0x7F, 0xFF) and c[0, 1] == 0 and c[0, 2] == 0x80 and c[0, 3] == 0
    sub = np.zeros((1, 32), np.uint16)
    sub[0, 0] = 0x0040  # bf16 subnormal 2^-127
    c, s = mo.cast_dim0(sub, mo.FLOOR)
    assert s[0, 0] == 0 and c[0, 0] == mo.e4m3_encode(np.array([0.5], np.float32))[0]
    c, s = mo.cast_dim0(sub, mo.RCEIL)
    assert s[0, 0] == 0 and c[0, 0] == 0


def test_exact_blocks_round_trip():
    """Blocks made of e4m3-representable values times a power of two survive cast -> dequant."""
    rng = np.random.default_rng(4)
    codes = rng.integers(0x08, 0x7F, size=(64, 64), dtype=np.uint8)  # normal codes
    codes[:, ::32] = 0x7E                                             # amax = 448 in every block
    codes |= rng.integers(0, 2, size=codes.shape, dtype=np.uint8) << 7
    scales = rng.integers(100, 150, size=(64, 2), dtype=np.uint8)
    x = mo.dequant(codes, scales)
    bits = mo.f32_to_bf16_bits(x)
    assert np.array_equal(mo.bf16_bits_to_f32(bits), x)  # 4 significant bits fit bf16
    for mode in (mo.FLOOR, mo.RCEIL):
        c, s = mo.cast_dim0(bits, mode)
        assert np.array_equal(c, codes) and np.array_equal(s, scales)


def test_c_restatement_agrees_on_random_bit_patterns():
    rng = np.random.default_rng(5)
    bits = rng.integers(0, 65536, size=(96, 256), dtype=np.uint16)
    blk = rng.integers(0, 65536, size=(2048, 32), dtype=np.uint16)
    blk[:, 0] = np.arange(0, 65536, 32, dtype=np.uint16)
    for mode in (mo.FLOOR, mo.RCEIL):
        for arr in (bits, blk):
            a, b = mo.cast_dim0(arr, mode), co.cast_dim0(arr, mode)
            assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
        a, b = mo.cast_dim1(bits, mode), co.cast_dim1(bits, mode)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    c, s = mo.cast_dim0(_cfg1_like(6, (32, 128)), mo.FLOOR)
    assert np.array_equal(mo.dequant(c, s), co.dequant(c, s))


# ------------------------------------------------------------------ matmul
def test_matmul_single_block_by_hand():
    """K = 32: A row = [2, 1, 0...], B row = [3, -1, 0...] -> exact dot 2*3 - 1 = 5."""
    a = np.zeros((1, 32), np.float32); a[0, :2] = [2, 1]
    b = np.zeros((1, 32), np.float32); b[0, :2] = [3, -1]
    for mode in (mo.FLOOR, mo.RCEIL):
        y = mo.mx_matmul(mo.f32_to_bf16_bits(a), mo.f32_to_bf16_bits(b), mode)
        assert mo.bf16_bits_to_f32(y)[0, 0] == 5.0


def test_matmul_vs_float64_and_textbook_dequant():
    rng = np.random.default_rng(7)
    a_bits, b_bits = _cfg1_like(8, (48, 256)), mo.f32_to_bf16_bits(rng.standard_normal((40, 256), dtype=np.float32) * 0.02)
    ac, asc = mo.cast_dim0(a_bits, mo.RCEIL)
    bc, bsc = mo.cast_dim0(b_bits, mo.RCEIL)
    # textbook dequant, element by element, independent of mo.dequant's vectorisation
    da = np.array([[mo.e4m3_decode(ac[r:r + 1, k:k + 1])[0, 0] * 2.0 ** (int(asc[r, k // 32]) - 127) for k in range(256)] for r in range(48)])
    assert np.array_equal(da.astype(np.float32), mo.dequant(ac, asc))
    ref = mo.f32_to_bf16_bits((da @ mo.dequant(bc, bsc).astype(np.float64).T).astype(np.float32))
    got = mo.mx_matmul_q(ac, asc, bc, bsc)
    diff = np.abs(mo.bf16_bits_to_f32(got).astype(np.float64) - mo.bf16_bits_to_f32(ref))
    assert np.linalg.norm(diff) / np.linalg.norm(mo.bf16_bits_to_f32(ref)) < 1e-3
    # MX matmul tracks the unquantized product to a few percent on N(0,1) x N(0,0.02) data
    exact = mo.bf16_bits_to_f32(a_bits).astype(np.float64) @ mo.bf16_bits_to_f32(b_bits).astype(np.float64).T
    rel = np.linalg.norm(mo.bf16_bits_to_f32(got) - exact) / np.linalg.norm(exact)
    assert rel < 0.06


def test_three_passes_are_transposes_of_one_primitive():
    rng = np.random.default_rng(9)
    x, w, dy = (mo.f32_to_bf16_bits(rng.standard_normal(s, dtype=np.float32)) for s in ((64, 96), (32, 96), (64, 32)))
    # dgrad == forward with W^T as the weight; wgrad == forward with dY^T as activation, X^T as weight
    assert np.array_equal(mo.linear_dgrad(dy, w), mo.linear_fwd(dy, np.ascontiguousarray(w.T)))
    assert np.array_equal(mo.linear_wgrad(dy, x), mo.linear_fwd(np.ascontiguousarray(dy.T), np.ascontiguousarray(x.T)))


def test_grouped_equals_loop_and_ignores_padding_rows():
    rng = np.random.default_rng(10)
    sizes = [32, 0, 96, 64]
    T = sum(sizes) + 32
    x = mo.f32_to_bf16_bits(rng.standard_normal((T, 64), dtype=np.float32))
    w = mo.f32_to_bf16_bits(rng.standard_normal((4, 48, 64), dtype=np.float32) * 0.1)
    y = mo.grouped_fwd(x, w, np.cumsum(sizes))
    assert np.all(y[sum(sizes):] == 0)
    assert np.array_equal(y[32:128], mo.linear_fwd(x[32:128], w[2]))
    dy = mo.f32_to_bf16_bits(rng.standard_normal((T, 48), dtype=np.float32))
    dw = mo.grouped_wgrad(dy, x, np.cumsum(sizes))
    assert np.all(dw[1] == 0) and np.array_equal(dw[3], mo.linear_wgrad(dy[128:192], x[128:192]))
    with pytest.raises(ValueError):
        mo.grouped_wgrad(dy, x, np.cumsum([16, 48, 96, 64]))


# ------------------------------------------------------------------ scale layout
def test_scale_layout_index_formula_and_round_trip():
    rng = np.random.default_rng(11)
    for rows, nblk in [(64, 4), (100, 7), (200, 13), (16, 1)]:
        s = rng.integers(1, 255, size=(rows, nblk), dtype=np.uint8)
        laid = mo.scale_layout(s)
        assert laid.shape == ((rows + 127) // 128, (nblk + 1) // 2, 64, 4)
        for _ in range(200):
            rt, ks, lane, t = (int(rng.integers(0, n)) for n in laid.shape)
            r, b = rt * 128 + t * 32 + (lane & 31), ks * 2 + (lane >> 5)
            assert laid[rt, ks, lane, t] == (s[r, b] if r < rows and b < nblk else 0)
        assert np.array_equal(mo.scale_unlayout(laid, rows, nblk), s)


# ------------------------------------------------------------------ group padding
def test_permute_indices_docstring_example_and_invariants():
    # torchtitan/models/common/moe/kernels.py:170-175: 2 ranks x 4 experts
    t = [4, 2, 1, 3, 1, 2, 3, 4]
    perm, m_sizes, m_offsets = mo.generate_permute_indices(t, 4, 2, 32, 8)
    assert m_sizes.tolist() == [8, 8, 8, 8] and m_offsets.tolist() == [8, 16, 24, 32]
    # expert 0 gets rank-0 tokens 0..3 then rank-1 token 10 (start of rank 1 / expert 0)
    assert perm[:8].tolist() == [0, 1, 2, 3, 10, -1, -1, -1]
    valid = perm[perm >= 0]
    assert sorted(valid.tolist()) == list(range(20))  # every routed token appears exactly once
    rng = np.random.default_rng(2020)
    for ranks in (1, 2, 8):
        experts = 64 // ranks
        for lo, hi in ((0, 0), (0, 5), (1, 16), (100, 300)):
            counts = rng.integers(lo, hi + 1, size=64)
            for A in (8, 16, 32):
                max_len = mo.padded_max_len(int(counts.sum()), experts, A)
                perm, ms, mofs = mo.generate_permute_indices(counts, experts, ranks, max_len, A)
                assert np.all(ms % A == 0) and np.all(ms >= A) and ms.dtype == np.int32
                tot = counts.reshape(ranks, -1).sum(0)
                wo = mofs - ms
                for e in range(experts):
                    seg = perm[wo[e]:mofs[e]]
                    assert np.all(seg[:tot[e]] >= 0) and np.all(seg[tot[e]:] == -1)
                assert sorted(perm[perm >= 0].tolist()) == list(range(int(counts.sum())))


def test_permute_indices_vs_host_reference_in_the_shell():
    from torchtitan_amd.modules import moe as moe_mod

    rng = np.random.default_rng(12)
    counts = rng.integers(0, 40, size=32)
    for ranks in (1, 4):
        experts = 32 // ranks
        perm, ms, mofs = mo.generate_permute_indices(counts, experts, ranks, 2048, 32)
        p2, ms2, mofs2 = moe_mod.generate_permute_indices(torch.from_numpy(counts), experts, ranks, 2048, 32, use_cpu=True)
        assert np.array_equal(perm, p2.numpy()) and np.array_equal(ms, ms2.numpy()) and np.array_equal(mofs, mofs2.numpy())


def test_cfg1_inputs_are_seeded_and_have_outliers():
    x, w = mo.make_cfg1_inputs(0, 256, 512, 128)
    x2, _ = mo.make_cfg1_inputs(0, 256, 512, 128)
    assert np.array_equal(x, x2) and x.shape == (256, 512) and w.shape == (128, 512)
    assert np.abs(mo.bf16_bits_to_f32(x)).max() > 20
