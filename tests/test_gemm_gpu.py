"""GPU parity: MXFP8 GEMM vs the oracle's emulated MX matmul (rel-L2 <= 1e-3, bf16 both sides)."""
import numpy as np
import pytest
import torch

from oracle import mx_oracle as mo
from tests.helpers import bf16_from_bits, bits_of, randn_bits, rel_l2, u8
from torchtitan_amd import _lib, ops

pytestmark = pytest.mark.gpu

TOL = 1e-3  # north-star tolerance: rel-L2, fp32 accumulate, bf16 out on both sides


def _gemm_from_codes(ac, asc, bc, bsc, device):
    a = ops.MXData(torch.from_numpy(ac).to(device), torch.from_numpy(asc).to(device), ops.MX_SCALES_ROWMAJOR)
    b = ops.MXData(torch.from_numpy(bc).to(device), torch.from_numpy(bsc).to(device), ops.MX_SCALES_ROWMAJOR)
    return ops.mx_gemm_nt(a, b)


def _f32(bits):
    return mo.bf16_bits_to_f32(bits)


@pytest.mark.parametrize("M,N,K", [(16, 16, 32), (16, 16, 128), (64, 64, 128), (128, 128, 256),
                                   (256, 256, 128), (256, 256, 512), (512, 768, 1024),
                                   (300, 200, 160), (257, 129, 96), (1000, 1000, 2048),
                                   (2048, 1024, 4096),
                                   # more tiles than workgroups, one or two K blocks per tile
                                   (4096, 4352, 128), (6144, 6400, 256)])
@pytest.mark.parametrize("force", [0, 3])
def test_gemm_matches_oracle(device, M, N, K, force):
    """force 0: the kernel the library picks for the shape; 3: the persistent kernel (mx_gemm32.hip)
    wherever it can run (small shapes would otherwise go to the tile kernel)."""
    from torchtitan_amd import _lib

    _lib.load().mx_debug_force_kernel(force)
    try:
        _check_gemm(device, M, N, K)
    finally:
        _lib.load().mx_debug_force_kernel(0)


def _check_gemm(device, M, N, K):
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    a_bits = randn_bits(rng, (M, K), outliers=1e-3)
    b_bits = randn_bits(rng, (N, K), std=0.02)
    ac, asc = mo.cast_dim0(a_bits, mo.FLOOR)
    bc, bsc = mo.cast_dim0(b_bits, mo.FLOOR)
    ref = mo.mx_matmul_q(ac, asc, bc, bsc)
    got = _gemm_from_codes(ac, asc, bc, bsc, device)
    err = rel_l2(_f32(bits_of(got)), _f32(ref))
    assert err <= TOL, f"rel-L2 {err}"


def test_one_hot_picks_single_products(device):
    """A = one-hot rows: D[m, n] must equal deq(A)[m, k_m] * deq(B)[n, k_m] rounded to bf16."""
    rng = np.random.default_rng(3)
    M, N, K = 128, 64, 256
    a = np.zeros((M, K), dtype=np.float32)
    ks = rng.integers(0, K, size=M)
    a[np.arange(M), ks] = rng.choice([1.0, -2.0, 0.5, 3.0], size=M)
    a_bits = mo.f32_to_bf16_bits(a)
    b_bits = randn_bits(rng, (N, K))
    ac, asc = mo.cast_dim0(a_bits, mo.RCEIL)
    bc, bsc = mo.cast_dim0(b_bits, mo.RCEIL)
    da, db = mo.dequant(ac, asc), mo.dequant(bc, bsc)
    expect = mo.f32_to_bf16_bits(da[np.arange(M), ks][:, None] * db[:, ks].T)
    got = bits_of(_gemm_from_codes(ac, asc, bc, bsc, device))
    assert np.array_equal(got, expect)


def test_unit_scales_reduce_to_plain_fp8(device):
    """All scale bytes 127: the result is the plain e4m3 x e4m3 product sum (exact in fp32 here)."""
    rng = np.random.default_rng(4)
    M, N, K = 64, 64, 128
    # normal codes in [2^-3, 1.875] with random signs: every partial sum is exact in fp32
    ac = rng.integers(0x20, 0x40, size=(M, K), dtype=np.uint8) | (rng.integers(0, 2, size=(M, K), dtype=np.uint8) << 7)
    bc = rng.integers(0x20, 0x40, size=(N, K), dtype=np.uint8) | (rng.integers(0, 2, size=(N, K), dtype=np.uint8) << 7)
    asc = np.full((M, K // 32), 127, dtype=np.uint8)
    bsc = np.full((N, K // 32), 127, dtype=np.uint8)
    ref = mo.f32_to_bf16_bits((mo.e4m3_decode(ac).astype(np.float64) @ mo.e4m3_decode(bc).astype(np.float64).T).astype(np.float32))
    got = bits_of(_gemm_from_codes(ac, asc, bc, bsc, device))
    assert np.array_equal(got, ref)


def test_scale_blocks_map_to_the_right_k(device):
    """Distinct power-of-two scale per (row, block): any mis-mapped scale changes the result."""
    M, N, K = 64, 32, 256
    ac = np.full((M, K), 0x38, dtype=np.uint8)  # 1.0
    bc = np.full((N, K), 0x38, dtype=np.uint8)
    asc = (120 + (np.arange(M)[:, None] % 5) + np.arange(K // 32)[None, :]).astype(np.uint8)
    bsc = (118 + (np.arange(N)[:, None] % 3) * 2 + (np.arange(K // 32)[None, :] % 4)).astype(np.uint8)
    ref = mo.mx_matmul_q(ac, asc, bc, bsc, accumulate=np.float64)
    got = bits_of(_gemm_from_codes(ac, asc, bc, bsc, device))
    assert np.array_equal(got, ref)


def test_each_scale_block_applies_to_its_own_32_k(device):
    """One-hot A at column k with per-block scales 127+b: D must be 2^(k // 32)."""
    M, N, K = 16, 16, 256
    for k in range(0, K, 8):
        ac = np.zeros((M, K), dtype=np.uint8)
        ac[:, k] = 0x38
        bc = np.full((N, K), 0x38, dtype=np.uint8)
        asc = np.tile((127 + np.arange(K // 32))[None, :], (M, 1)).astype(np.uint8)
        bsc = np.full((N, K // 32), 127, dtype=np.uint8)
        got = _f32(bits_of(_gemm_from_codes(ac, asc, bc, bsc, device)))
        assert np.all(got == 2.0 ** (k // 32)), k
        got = _f32(bits_of(_gemm_from_codes(bc, bsc, ac, asc, device)))
        assert np.all(got == 2.0 ** (k // 32)), k


def test_linear_passes_end_to_end(device):
    """fwd, dgrad, wgrad built from the HIP casts + GEMM vs the oracle's three passes."""
    rng = np.random.default_rng(5)
    M, K, N = 512, 256, 384
    x_bits = randn_bits(rng, (M, K), outliers=1e-3)
    w_bits = randn_bits(rng, (N, K), std=0.02)
    dy_bits = randn_bits(rng, (M, N), std=1e-3)
    x, w, dy = (bf16_from_bits(b, device) for b in (x_bits, w_bits, dy_bits))
    L = ops.MX_SCALES_MFMA
    for mode_name, mode in (("floor", mo.FLOOR), ("rceil", mo.RCEIL)):
        y = ops.mx_gemm_nt(ops.to_mx_dim0(x, mode_name, L), ops.to_mx_dim0(w, mode_name, L))
        dx = ops.mx_gemm_nt(ops.to_mx_dim0(dy, mode_name, L), ops.to_mx_dim1(w, mode_name, L))
        dw = ops.mx_gemm_nt(ops.to_mx_dim1(dy, mode_name, L), ops.to_mx_dim1(x, mode_name, L))
        assert rel_l2(_f32(bits_of(y)), _f32(mo.linear_fwd(x_bits, w_bits, mode))) <= TOL
        assert rel_l2(_f32(bits_of(dx)), _f32(mo.linear_dgrad(dy_bits, w_bits, mode))) <= TOL
        assert rel_l2(_f32(bits_of(dw)), _f32(mo.linear_wgrad(dy_bits, x_bits, mode))) <= TOL


def test_full_size_linearity(device):
    """8B-FFN shape: D(A, B) rows are independent and scale-linear.

    Doubling every A scale byte (+1) must exactly double D (power-of-two scaling commutes with
    fp32 accumulation and bf16 rounding), and a row slice of the big GEMM must equal the GEMM of
    the slice -- both hold for any correct kernel at any size, without a CPU pass.
    """
    torch.manual_seed(1)
    M, K, N = 16384, 4096, 14336
    x = torch.randn((M, K), device=device, dtype=torch.bfloat16)
    w = torch.randn((N, K), device=device, dtype=torch.bfloat16) * 0.02
    a = ops.to_mx_dim0(x, "floor")
    b = ops.to_mx_dim0(w, "floor")
    d = ops.mx_gemm_nt(a, b)
    a2 = ops.MXData(a.codes, a.scales + 1, a.scale_order)
    d2 = ops.mx_gemm_nt(a2, b)
    assert torch.equal(d2, d * 2)
    rows = slice(5000, 5000 + 192)
    ds = ops.mx_gemm_nt(ops.MXData(a.codes[rows].contiguous(), a.scales[rows].contiguous(), a.scale_order), b)
    assert torch.equal(ds, d[rows])
    # a 64x96 corner against the oracle
    ref = mo.mx_matmul_q(u8(a.codes[:64]), u8(a.scales[:64]), u8(b.codes[:96]), u8(b.scales[:96]))
    err = rel_l2(_f32(bits_of(d[:64, :96])), _f32(ref))
    assert err <= TOL


def test_config1_full_size_against_the_oracle(device):
    """The CPU-runnable baseline config at its full size: X[8192,4096], W[4096,4096] with 0.1 %
    x100 outliers, FLOOR and RCEIL: codes and scales of all four casts bit-exact against the C
    oracle, Y against the oracle's dequantize + fp32 matmul + bf16 round (rel-L2 <= 1e-3)."""
    from oracle import c_oracle as co

    x_bits, w_bits = mo.make_cfg1_inputs(0)
    x, w = bf16_from_bits(x_bits, device), bf16_from_bits(w_bits, device)
    R = ops.MX_SCALES_ROWMAJOR
    for mode_name, mode in (("floor", mo.FLOOR), ("rceil", mo.RCEIL)):
        for t_bits, t in ((x_bits, x), (w_bits, w)):
            q0, q1 = ops.to_mx_dim0_dim1(t, mode_name, R)
            c0, s0 = co.cast_dim0(t_bits, mode)
            c1, s1 = co.cast_dim1(t_bits, mode)
            assert np.array_equal(u8(q0.codes), c0) and np.array_equal(u8(q0.scales), s0)
            assert np.array_equal(u8(q1.codes), c1) and np.array_equal(u8(q1.scales), s1)
        L = ops.MX_SCALES_MFMA
        y = ops.mx_gemm_nt(ops.to_mx_dim0(x, mode_name, L), ops.to_mx_dim0(w, mode_name, L))
        xc, xs = co.cast_dim0(x_bits, mode)
        wc, ws = co.cast_dim0(w_bits, mode)
        ref = mo.f32_to_bf16_bits(co.dequant(xc, xs) @ co.dequant(wc, ws).T)
        assert rel_l2(_f32(bits_of(y)), _f32(ref)) <= TOL


@pytest.mark.parametrize("M,N,K", [(512, 384, 256), (96, 80, 64), (1024, 1000, 128)])
def test_output_row_stride(device, M, N, K):
    """D may be a column slice of a wider buffer (ldd > N): nothing outside the slice is touched."""
    rng = np.random.default_rng(M + N + K)
    a_bits = randn_bits(rng, (M, K), outliers=1e-3)
    b_bits = randn_bits(rng, (N, K), std=0.02)
    ac, asc = mo.cast_dim0(a_bits, mo.RCEIL)
    bc, bsc = mo.cast_dim0(b_bits, mo.RCEIL)
    ref = mo.mx_matmul_q(ac, asc, bc, bsc)
    a = ops.to_mx_dim0(bf16_from_bits(a_bits, device), "rceil")
    b = ops.to_mx_dim0(bf16_from_bits(b_bits, device), "rceil")
    wide = torch.full((M, N + 56), 7.0, dtype=torch.bfloat16, device=device)
    ops.mx_gemm_nt(a, b, out=wide[:, 24:24 + N])
    assert rel_l2(_f32(bits_of(wide[:, 24:24 + N].contiguous())), _f32(ref)) <= TOL
    assert torch.all(wide[:, :24] == 7.0) and torch.all(wide[:, 24 + N:] == 7.0)


@pytest.mark.parametrize("M,N,K", [(512, 512, 16384),    # 4 tiles, 128 K blocks
                                   (700, 520, 16384),    # ragged tile edges
                                   (768, 256, 12288 + 128)])  # 97 blocks: slices of unequal length
def test_gemm_split_along_k_matches_oracle(device, M, N, K):
    """Few output tiles and a long contraction: the library splits K over several workgroups per
    tile (float32 partial sums in a workspace, one reduction).  Against the oracle, and against
    the unsplit call: the two differ only by float32 summation order."""
    from torchtitan_amd import _lib

    lib = _lib.load()
    with torch.cuda.device(device):
        need = int(lib.mx_gemm_nt_workspace_bytes(M, N, K))
    assert need > 0 and need % (M * N * 4) == 0, "the shape is meant to be split"
    rng = np.random.default_rng(M + N + K)
    a_bits = randn_bits(rng, (M, K), outliers=1e-3)
    b_bits = randn_bits(rng, (N, K), std=0.02)
    ac, asc = mo.cast_dim0(a_bits, mo.FLOOR)
    bc, bsc = mo.cast_dim0(b_bits, mo.FLOOR)
    ref = _f32(mo.mx_matmul_q(ac, asc, bc, bsc))
    a = ops.MXData(torch.from_numpy(ac).to(device), torch.from_numpy(asc).to(device), ops.MX_SCALES_ROWMAJOR)
    b = ops.MXData(torch.from_numpy(bc).to(device), torch.from_numpy(bsc).to(device), ops.MX_SCALES_ROWMAJOR)
    launches = []
    real_call = ops._call
    ops._call = lambda name, *rest: (launches.append(name), real_call(name, *rest))[1]
    try:
        got = ops.mx_gemm_nt(a, b)
        wide = torch.full((M, N + 24), 7.0, dtype=torch.bfloat16, device=device)
        ops.mx_gemm_nt(a, b, out=wide[:, :N])  # row stride larger than N
    finally:
        ops._call = real_call
    assert launches.count("mx_gemm_nt_ws") == 2
    assert rel_l2(_f32(bits_of(got)), ref) <= TOL
    assert torch.equal(wide[:, :N], got) and bool((wide[:, N:] == 7.0).all())
    # the unsplit kernel on the same operands
    sa, sb = ops._as_mfma(a), ops._as_mfma(b)
    plain = torch.empty_like(got)
    real_call("mx_gemm_nt", "gemm_nt", got.device, ops._ptr(a.codes), ops._ptr(sa), ops._ptr(b.codes),
              ops._ptr(sb), ops._ptr(plain), M, N, K, N, ops._stream(plain))
    assert rel_l2(got.float().cpu().numpy(), plain.float().cpu().numpy()) <= 3e-4
    # without the workspace (or with too little of it) the call is the unsplit one
    for ws, nbytes in ((None, 0), (torch.empty(need // 2, dtype=torch.uint8, device=device), need // 2)):
        again = torch.empty_like(got)
        real_call("mx_gemm_nt_ws", "gemm_nt_ws", got.device, ops._ptr(a.codes), ops._ptr(sa), ops._ptr(b.codes),
                  ops._ptr(sb), ops._ptr(again), M, N, K, N, ops._ptr(ws) if ws is not None else None, nbytes,
                  ops._stream(again))
        assert torch.equal(again, plain)


@pytest.mark.parametrize("M,N,K", [(256, 256, 512), (1024, 768, 4096), (4096, 1024, 1024)])
def test_gemm_agrees_with_the_vendor_block_scaled_gemm(device, M, N, K):
    """An implementation of the same contract that shares nothing with this repository: the
    vendor library's MX block-scaled GEMM behind torch._scaled_mm (e4m3 operands, one E8M0 scale
    per 32 elements along K, row-major scale matrices) -- the call the reference's path ends in
    (docs/mxfp8.md:36).  Operands with block scales spread over 2^-6 .. 2^5, so a scale applied
    to the wrong block or read from the wrong byte would be far off.  The vendor kernel is asked
    for fp16 output (it rounds that to nearest; its bf16 output is truncated, one step below
    round-to-nearest on half of the elements).  Against that finer result this kernel's bf16
    output may be off by its own rounding only: rel-L2 <= 2.5e-3 (bf16 rounding noise is about
    1.5e-3); rounded on to bf16 the vendor result is the same number at more than 9 elements in
    10 and never more than one bf16 step away (double rounding and summation order)."""
    torch.manual_seed(M + K)

    def spread(rows, lo, hi):  # one power of two per 32-element block
        e = torch.randint(lo, hi, (rows, K // 32), device=device).repeat_interleave(32, 1)
        return torch.exp2(e.float()).to(torch.bfloat16)

    x = torch.randn(M, K, device=device, dtype=torch.bfloat16) * spread(M, -6, 6)
    w = torch.randn(N, K, device=device, dtype=torch.bfloat16) * 0.02 * spread(N, -4, 4)
    xq = ops.to_mx_dim0(x, "rceil", ops.MX_SCALES_ROWMAJOR)
    wq = ops.to_mx_dim0(w, "rceil", ops.MX_SCALES_ROWMAJOR)
    mine = ops.mx_gemm_nt(xq, wq)
    try:
        vendor = torch._scaled_mm(xq.codes.view(torch.float8_e4m3fn), wq.codes.view(torch.float8_e4m3fn).t(),
                                  scale_a=xq.scales.view(torch.float8_e8m0fnu),
                                  scale_b=wq.scales.view(torch.float8_e8m0fnu), out_dtype=torch.float16)
    except (RuntimeError, ValueError, NotImplementedError) as ex:
        pytest.skip(f"this torch build has no MX block-scaled GEMM: {ex}")
    want = vendor.float().to(torch.bfloat16)
    assert rel_l2(mine.float().cpu().numpy(), vendor.float().cpu().numpy()) <= 2.5e-3
    steps = (mine.view(torch.int16).int() - want.view(torch.int16).int()).abs()
    normal = vendor.abs() >= 2.0 ** -13  # below that fp16 itself is coarser than bf16
    assert int(steps[normal].max()) <= 1 and float((steps == 0).float().mean()) > 0.9


def test_policy_step_token_count_row_blocks_equal_small_calls(device):
    """147 456 packed tokens (the policy step of the RL config) against a 2048 -> 6144 projection:
    far beyond what the oracle can do, but every block of rows of the cast and of the GEMM
    depends on those rows only.  Blocks from the start, the middle and the very end of the token
    axis must equal the same kernels run on that slice alone, bit for bit; the weight gradient
    over all tokens (split along K) must equal the sum of the gradients over two halves to
    float32-summation accuracy."""
    T, K, N = 147456, 2048, 6144
    torch.manual_seed(11)
    x = torch.randn(T, K, device=device, dtype=torch.bfloat16)
    w = torch.randn(N, K, device=device, dtype=torch.bfloat16) * 0.02
    xq0, xq1 = ops.to_mx_dim0_dim1(x, "rceil", ops.MX_SCALES_MFMA)
    wq0 = ops.to_mx_dim0(w, "rceil", ops.MX_SCALES_MFMA)
    y = ops.mx_gemm_nt(xq0, wq0)
    for r0 in (0, 73728 - 128, T - 512):
        part = x[r0:r0 + 512].contiguous()
        pq0, pq1 = ops.to_mx_dim0_dim1(part, "rceil", ops.MX_SCALES_MFMA)
        assert torch.equal(xq0.codes[r0:r0 + 512], pq0.codes)
        assert torch.equal(xq1.codes[:, r0:r0 + 512], pq1.codes)
        assert torch.equal(y[r0:r0 + 512], ops.mx_gemm_nt(pq0, wq0)), r0
    del y
    dy = torch.randn(T, 1024, device=device, dtype=torch.bfloat16) * 1e-3
    dyq1 = ops.to_mx_dim1(dy, "rceil", ops.MX_SCALES_MFMA)
    dw = ops.mx_gemm_nt(dyq1, xq1)  # [1024, 2048] over 147 456 tokens: split along K
    halves = torch.zeros_like(dw, dtype=torch.float32)
    for r0 in (0, T // 2):
        a = ops.to_mx_dim1(dy[r0:r0 + T // 2].contiguous(), "rceil", ops.MX_SCALES_MFMA)
        b = ops.to_mx_dim1(x[r0:r0 + T // 2].contiguous(), "rceil", ops.MX_SCALES_MFMA)
        halves += ops.mx_gemm_nt(a, b).float()
    # each half is rounded to bf16 before the sum: two roundings of 2^-9 relative against one
    assert rel_l2(dw.float().cpu().numpy(), halves.cpu().numpy()) <= 3e-3


@pytest.mark.parametrize("M,N,K", [(512, 384, 256), (300, 264, 128), (1024, 1024, 1024), (2048, 4096, 512)])
def test_pair_gemm_is_one_gemm_over_the_concatenated_contraction(device, M, N, K):
    """D = A B^T + A2 B2^T in one pass equals the oracle's MX matmul of [A | A2] with [B | B2]
    (one rounding to bf16), and is at least as close to it as two GEMMs and a bf16 add."""
    rng = np.random.default_rng(M + 3 * N + K)
    ops_q = []
    for std in (1.0, 0.02, 0.5, 0.05):
        rows = M if len(ops_q) % 2 == 0 else N
        ops_q.append(mo.cast_dim0(randn_bits(rng, (rows, K), std=std), mo.RCEIL))
    (ac, asc), (bc, bsc), (a2c, a2sc), (b2c, b2sc) = ops_q
    ref = _f32(mo.mx_matmul_q(np.concatenate([ac, a2c], 1), np.concatenate([asc, a2sc], 1),
                              np.concatenate([bc, b2c], 1), np.concatenate([bsc, b2sc], 1)))
    dev = lambda c, s_: ops.MXData(torch.from_numpy(c).to(device), torch.from_numpy(s_).to(device), ops.MX_SCALES_ROWMAJOR)
    a, b, a2, b2 = dev(ac, asc), dev(bc, bsc), dev(a2c, a2sc), dev(b2c, b2sc)
    launches = []
    real_call = ops._call
    ops._call = lambda name, *rest: (launches.append(name), real_call(name, *rest))[1]
    try:
        got = ops.mx_gemm_nt_pair(a, b, a2, b2)
    finally:
        ops._call = real_call
    assert launches.count("mx_gemm_nt_pair_ld") == 1 and "mx_gemm_nt" not in launches
    err = rel_l2(_f32(bits_of(got)), ref)
    two = ops.mx_gemm_nt(a, b) + ops.mx_gemm_nt(a2, b2)
    assert err <= TOL and err <= rel_l2(_f32(bits_of(two)), ref) + 1e-5, err


def _launch_names(fn):
    """(result of fn(), names of the C-ABI entry points it called)."""
    names = []
    real_call = ops._call
    ops._call = lambda name, *rest: (names.append(name), real_call(name, *rest))[1]
    try:
        return fn(), names
    finally:
        ops._call = real_call


@pytest.mark.parametrize("M,N,K", [(512, 384, 256), (300, 264, 128), (2304, 1280, 512), (1024, 4096, 1024)])
def test_two_products_sharing_an_operand_equal_two_gemms(device, M, N, K):
    """One launch for A B^T and A B2^T (and for A B^T and A2 B^T): every tile is computed as by
    mx_gemm_nt, so both outputs equal the separate calls bit for bit; and against the oracle."""
    rng = np.random.default_rng(7 * M + N + K)
    q = lambda rows, std: ops.to_mx_dim0(bf16_from_bits(randn_bits(rng, (rows, K), std=std), device), "rceil",
                                         ops.MX_SCALES_MFMA)
    a, a2, b, b2 = q(M, 1.0), q(M, 0.3), q(N, 0.02), q(N, 0.05)
    (d, d2), names = _launch_names(lambda: ops.mx_gemm_nt_shared_a(a, b, b2))
    assert names == ["mx_gemm_nt_shared_a_ld"]
    assert torch.equal(d, ops.mx_gemm_nt(a, b)) and torch.equal(d2, ops.mx_gemm_nt(a, b2))
    (e, e2), names = _launch_names(lambda: ops.mx_gemm_nt_shared_b(a, a2, b))
    assert names == ["mx_gemm_nt_shared_b_ld"]
    assert torch.equal(e, d) and torch.equal(e2, ops.mx_gemm_nt(a2, b))
    # the same on operands whose rows lie 128 bytes further apart (NaN codes between the rows), and the
    # sum of two products likewise: bit-identical; one operand with another pitch: copies, then dense
    def pitched(t, pad=128):
        buf = torch.full((t.codes.shape[0], K + pad), 0x7F, dtype=torch.uint8, device=device)
        buf[:, :K] = t.codes
        return ops.MXData(buf[:, :K], t.scales, t.scale_order)

    pa, pa2, pb, pb2 = pitched(a), pitched(a2), pitched(b), pitched(b2)
    assert torch.equal(ops.mx_gemm_nt_shared_a(pa, pb, pb2), torch.stack((d, d2)))
    assert torch.equal(ops.mx_gemm_nt_shared_b(pa, pa2, pb), torch.stack((e, e2)))
    assert torch.equal(ops.mx_gemm_nt_shared_a(pa, pb, b2), torch.stack((d, d2)))
    both = ops.mx_gemm_nt_pair(a, b, a2, b2)
    assert torch.equal(ops.mx_gemm_nt_pair(pa, pb, pa2, pb2), both)
    assert torch.equal(ops.mx_gemm_nt_pair(pa, pb, pa2, pitched(b2, 256)), both)
    un = lambda t: ops.scale_unlayout(t.scales, t.codes.shape[0], K // 32).cpu().numpy()
    ref = mo.mx_matmul_q(a2.codes.cpu().numpy(), un(a2), b.codes.cpu().numpy(), un(b))
    assert rel_l2(_f32(bits_of(e2)), _f32(ref)) <= TOL


def test_two_products_fall_back_to_two_gemms_on_small_shapes(device):
    rng = np.random.default_rng(5)
    q = lambda rows: ops.to_mx_dim0(bf16_from_bits(randn_bits(rng, (rows, 96)), device), "rceil", ops.MX_SCALES_MFMA)
    a, b, b2 = q(64), q(40), q(40)
    (d, d2), names = _launch_names(lambda: ops.mx_gemm_nt_shared_a(a, b, b2))
    assert names == ["mx_gemm_nt", "mx_gemm_nt"]
    assert torch.equal(d, ops.mx_gemm_nt(a, b)) and torch.equal(d2, ops.mx_gemm_nt(a, b2))


@pytest.mark.parametrize("M,N,K", [(512, 384, 256), (300, 264, 128), (96, 64, 160), (2048, 1024, 4096), (768, 256, 16384)])
def test_gemm_on_operands_with_a_row_pitch_equals_the_dense_gemm(device, M, N, K):
    """Operand rows 128 bytes further apart than they are long (what the fused cast writes for the
    dense linear): the same kernels on the same values, so bit-identical to dense operands, on the
    persistent kernel, its split form and the small-shape tile kernels alike; operands whose
    pitches differ are brought to one."""
    rng = np.random.default_rng(M + N + K)
    a = ops.to_mx_dim0(bf16_from_bits(randn_bits(rng, (M, K), outliers=1e-3), device), "rceil", ops.MX_SCALES_MFMA)
    b = ops.to_mx_dim0(bf16_from_bits(randn_bits(rng, (N, K), std=0.02), device), "rceil", ops.MX_SCALES_MFMA)
    want = ops.mx_gemm_nt(a, b)

    def pitched(d, pad):
        buf = torch.full((d.codes.shape[0], K + pad), 0x7F, dtype=torch.uint8, device=device)  # NaN codes between the rows
        buf[:, :K] = d.codes
        return ops.MXData(buf[:, :K], d.scales, d.scale_order)

    (got, names) = _launch_names(lambda: ops.mx_gemm_nt(pitched(a, 128), pitched(b, 128)))
    assert names == ["mx_gemm_nt_ld"] and torch.equal(got, want)
    assert torch.equal(ops.mx_gemm_nt(pitched(a, 128), b), want)  # differing pitches: copies, then dense
    # a pitch that is not a multiple of 128: the tile kernel, which never splits the contraction
    odd = ops.mx_gemm_nt(pitched(a, 16), pitched(b, 16))
    with torch.cuda.device(device):
        split = int(_lib.load().mx_gemm_nt_workspace_bytes(M, N, K)) > 0
    if split:
        assert rel_l2(odd.float().cpu().numpy(), want.float().cpu().numpy()) <= 3e-4
    else:
        assert torch.equal(odd, want)
