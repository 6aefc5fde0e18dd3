"""CPU oracle for the MXFP8 linear path.  TEST INFRASTRUCTURE ONLY.

This module is the checker for the HIP kernels: only tests, the smoke check and the
benchmark's CPU-baseline leg may import it.  The product never routes through it.

It restates, in NumPy integer/float32 arithmetic, the path that the reference's MXFP8
converter hands to an external library (reference call site:
torchtitan/components/quantization/mx.py:100-125; format statement docs/mxfp8.md:31-37;
block-size constant torchtitan/components/quantization/__init__.py:36).  That library
(torchao, unpinned: "--pre" nightly in .github/workflows/unit_test_cpu.yaml:33,
"v0.14.0 or newer" in docs/mxfp8.md:27) is absent from the reference tree, so every
function here is written from the OCP Microscaling (MX) v1.0 block format:

  * element type  e4m3fn : S EEEE MMM, bias 7, max 448, no inf, 0x7F/0xFF = NaN
  * scale type    E8M0   : byte b means 2**(b-127), b = 255 means NaN
  * block         32 consecutive elements along the contraction dim share one scale

Pinning status (what fixes each function independently of its own formula):

  e4m3_encode / e4m3_decode  pinned  -- torch's CPU float8_e4m3fn cast (library routine),
                                        exhaustive over all bf16 inputs; decode/encode
                                        round trip over all 256 codes
  bf16 <-> f32               pinned  -- torch's CPU bfloat16 cast, exhaustive
  scale byte FLOOR / RCEIL   pinned for finite normal amax by the closed forms
                                        floor(log2 amax) - 8 and ceil(log2(amax/448))
                                        evaluated in float64 over every bf16 amax, plus the
                                        hand-computed known answers in tests/golden
                             PARITY UNPINNED for: amax = 0 / subnormal / inf / NaN, the
                                        clamp of the scale byte at 0, and which of
                                        FLOOR / RCEIL the reference recipe means at a given
                                        call site (the converter asks for "mxfp8_rceil",
                                        mx.py:37-42); no reference test holds a vector
  cast_dim1                  pinned  -- by definition equal to cast_dim0 of the transpose
  mx_matmul                  pinned  -- textbook: exact dequantize, float64 matmul, special
                                        cases (unit scales, one-hot operands, K = 32)
  grouped variants           pinned  -- loop of mx_matmul over groups, the shape of the
                                        reference's own per-expert loop
                                        (torchtitan/models/common/moe/moe.py:24-56)
  rms_norm_bf16              pinned  -- textbook form in float64 vs torch's CPU rms_norm; last bf16
                                        step under a float32 reduction PARITY UNPINNED
  swiglu_bf16                pinned  -- closed form in float64; the last bf16 ulp of a
                                        float32 evaluation is PARITY UNPINNED (see its docstring)
  swiglu_backward_bf16       pinned  -- closed form vs a central difference and torch's CPU op;
                                        last bf16 ulp of da PARITY UNPINNED (see its docstring)
  moe_route_plan             pinned  -- composition of generate_permute_indices (pinned) with index
                                        arithmetic; checked against torch indexing in the tests
  gather_rows                pinned  -- index semantics vs torch indexing; score product exact
                                        before its bf16 rounding (torch CPU ops)
  moe_combine                pinned  -- vs an exact float64 sum (within one bf16 step) and torch's
                                        scatter + bmm on the CPU; accumulation order PARITY UNPINNED
  moe_row_dot                pinned  -- float64 dot products (textbook)
  token_log_probs(_grad)     pinned  -- torch CPU float32 log_softmax + gather and its autograd
  policy_gradient_loss       pinned  -- closed forms (policy == reference; hand example) and the
                                        formulas run with torch ops on the CPU
  generate_permute_indices   pinned  -- the worked example and invariants of
                                        torchtitan/models/common/moe/kernels.py:145-218
                                        and tests/unit_tests/test_permute_indices_kernel.py

bf16 tensors are carried as uint16 bit patterns, fp8 codes and scales as uint8.
"""
from __future__ import annotations

import numpy as np

BLOCK = 32  # torchtitan/components/quantization/__init__.py:36 (MXFP8_GROUP_ALIGNMENT_SIZE)
FLOOR = 0
RCEIL = 1
E4M3_MAX = 448.0
E4M3_EMAX = 8  # 448 = 1.75 * 2**8


# --------------------------------------------------------------------------- formats
def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    """bf16 is the top half of an IEEE float32."""
    return (np.ascontiguousarray(bits).astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even narrowing of float32 to bf16 bit patterns (NaN stays NaN)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    r = ((u.astype(np.uint64) + np.uint64(0x7FFF) + lsb) >> np.uint64(16)).astype(np.uint16)
    quiet = ((u >> np.uint32(16)) | np.uint32(0x0040)).astype(np.uint16)
    return np.where(nan, quiet, r)


def e4m3_decode_table() -> np.ndarray:
    """Value of each of the 256 e4m3fn codes, from the format definition."""
    t = np.zeros(256, dtype=np.float32)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 0x7
        if e == 0xF and m == 0x7:
            v = float("nan")
        elif e == 0:
            v = s * m * 2.0 ** -9
        else:
            v = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
        t[c] = v
    return t


_E4M3_TABLE = e4m3_decode_table()


def e4m3_decode(codes: np.ndarray) -> np.ndarray:
    return _E4M3_TABLE[codes]


def e4m3_encode(y: np.ndarray) -> np.ndarray:
    """Saturating round-to-nearest-even narrowing float32 -> e4m3fn code.

    |y| > 448 (inf included) saturates to 0x7E; NaN gives 0x7F; the sign bit is kept,
    so -0.0 gives 0x80.
    """
    y = np.ascontiguousarray(y, dtype=np.float32)
    u = y.view(np.uint32)
    sign = ((u >> np.uint32(24)) & np.uint32(0x80)).astype(np.uint8)
    a = u & np.uint32(0x7FFFFFFF)
    nan = a > np.uint32(0x7F800000)
    a = np.minimum(a, np.uint32(0x43E00000))  # 448.0f
    # normal e4m3 range: keep 3 mantissa bits with ties-to-even, then rebias 127 -> 7
    lsb = (a >> np.uint32(20)) & np.uint32(1)
    rn = (a + np.uint32(0x7FFFF) + lsb) >> np.uint32(20)
    normal = (rn - np.uint32(120 << 3)).astype(np.int64)
    # below 2**-6 the code is the integer number of 2**-9 steps, ties-to-even
    mag = a.view(np.float32)
    sub = np.rint(mag * np.float32(512.0)).astype(np.int64)
    code = np.where(a < np.uint32(0x3C800000), sub, normal)
    code = np.where(nan, 0x7F, code).astype(np.uint8)
    return code | sign


# --------------------------------------------------------------------------- scales
def scale_from_amax_bits(amax_bits: np.ndarray, mode: int) -> np.ndarray:
    """E8M0 byte for a block whose max |x| has bf16 bit pattern `amax_bits` (sign clear).

    FLOOR: s = floor(log2 amax) - 8, read off the exponent field.
    RCEIL: s = ceil(log2(amax / 448)) = E - 8 + [mantissa > 0.75] for amax = (1+m) 2**E.
    Both clamp s to [-127, 127]; byte = s + 127; NaN amax -> 255; amax = 0 -> 0.
    Unpinned corners, fixed here: a subnormal amax is treated as E = -127 (FLOOR) or by
    its true log2 (RCEIL, always clamps to byte 0); amax = inf follows the same integer
    formula as a finite value with exponent field 255.
    """
    a = amax_bits.astype(np.int64)
    expf = a >> 7
    man = a & 0x7F
    if mode == FLOOR:
        s = expf - 127 - E4M3_EMAX
    elif mode == RCEIL:
        s = expf - 127 - E4M3_EMAX + (man > 0x60)
    else:
        raise ValueError(f"unknown scale mode {mode}")
    s = np.clip(s, -127, 127)
    byte = s + 127
    byte = np.where(a == 0, 0, byte)
    byte = np.where(a > 0x7F80, 255, byte)
    return byte.astype(np.uint8)


def _multiplier_from_scale(byte: np.ndarray, mode: int) -> np.ndarray:
    """float32 factor 2**(-s) applied to the block before narrowing.

    For byte 0 the factor is 2**126 in FLOOR mode (the divisor is held at the smallest
    normal float32) and 1.0 in RCEIL mode; both only reachable for amax <= 2**-119.
    For byte 255 (NaN block) the factor is 0, so finite lanes become signed zeros and
    NaN lanes stay NaN.
    """
    b = byte.astype(np.int64)
    e = 127 - b  # -s
    mult_bits = ((e + 127) << 23).astype(np.uint32)
    mult = mult_bits.view(np.float32).copy()
    if mode == FLOOR:
        mult = np.where(b == 0, np.float32(2.0 ** 126), mult)
    else:
        mult = np.where(b == 0, np.float32(1.0), mult)
    mult = np.where(b == 254, np.float32(2.0 ** -127), mult)  # subnormal factor
    mult = np.where(b == 255, np.float32(0.0), mult)
    return mult.astype(np.float32)


# --------------------------------------------------------------------------- casts
def cast_dim0(x_bits: np.ndarray, mode: int = FLOOR):
    """Row-wise to_mx: bf16 [R, C] -> (codes u8 [R, C], scales u8 [R, C/32]).

    Blocks of 32 run along the last (contiguous) dimension.
    """
    x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
    R, C = x_bits.shape
    if C % BLOCK:
        raise ValueError("last dim must be a multiple of 32")
    blk = x_bits.reshape(R, C // BLOCK, BLOCK)
    amax_bits = (blk & np.uint16(0x7FFF)).max(axis=-1)
    scales = scale_from_amax_bits(amax_bits, mode)
    mult = _multiplier_from_scale(scales, mode)
    with np.errstate(invalid="ignore", over="ignore"):
        y = bf16_bits_to_f32(blk) * mult[..., None]
    # inf * 0 above would give NaN for an inf lane in a NaN block; keep it a signed zero
    inf_lane = (blk & np.uint16(0x7FFF)) == np.uint16(0x7F80)
    nan_blk = (scales == 255)[..., None]
    y = np.where(inf_lane & nan_blk, np.copysign(np.float32(0), bf16_bits_to_f32(blk)), y)
    codes = e4m3_encode(y.astype(np.float32)).reshape(R, C)
    return codes, scales


def cast_dim1(x_bits: np.ndarray, mode: int = FLOOR):
    """Column-wise to_mx: bf16 [R, C] -> (codes u8 [C, R], scales u8 [C, R/32]).

    Blocks of 32 run down the first dimension; outputs are stored transposed so the
    quantized axis is contiguous.
    """
    return cast_dim0(np.ascontiguousarray(np.asarray(x_bits).T), mode)


def dequant(codes: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """float32 value of MX data: e4m3 value times 2**(scale-127), blocks along last dim."""
    R, C = codes.shape
    v = e4m3_decode(codes).reshape(R, C // BLOCK, BLOCK).astype(np.float64)
    s = np.where(scales == 255, np.nan, np.exp2(scales.astype(np.float64) - 127.0))
    return (v * s[..., None]).reshape(R, C).astype(np.float32)


# --------------------------------------------------------------------------- matmul
def mx_matmul_q(a_codes, a_scales, b_codes, b_scales, accumulate=np.float32) -> np.ndarray:
    """bf16 bits of  deq(A)[M,K] @ deq(B)[N,K]^T  with `accumulate`-precision sums."""
    a = dequant(a_codes, a_scales).astype(accumulate)
    b = dequant(b_codes, b_scales).astype(accumulate)
    return f32_to_bf16_bits((a @ b.T).astype(np.float32))


def mx_matmul(a_bits: np.ndarray, b_bits: np.ndarray, mode: int = FLOOR, accumulate=np.float32):
    """Emulated MXFP8 product of bf16 A[M,K] and B[N,K], both quantized along K."""
    ac, asc = cast_dim0(a_bits, mode)
    bc, bsc = cast_dim0(b_bits, mode)
    return mx_matmul_q(ac, asc, bc, bsc, accumulate)


def linear_fwd(x_bits, w_bits, mode=FLOOR):
    """Y[M,N] = X[M,K] W[N,K]^T, both cast along K."""
    return mx_matmul(x_bits, w_bits, mode)


def linear_dgrad(dy_bits, w_bits, mode=FLOOR):
    """dX[M,K] = dY[M,N] W[N,K]: dY cast along N (dim0), W cast along N (dim1)."""
    ac, asc = cast_dim0(dy_bits, mode)
    bc, bsc = cast_dim1(w_bits, mode)
    return mx_matmul_q(ac, asc, bc, bsc)


def linear_wgrad(dy_bits, x_bits, mode=FLOOR):
    """dW[N,K] = dY[M,N]^T X[M,K]: both cast along M (dim1)."""
    ac, asc = cast_dim1(dy_bits, mode)
    bc, bsc = cast_dim1(x_bits, mode)
    return mx_matmul_q(ac, asc, bc, bsc)


# --------------------------------------------------------------------------- grouped
def _group_bounds(offs):
    offs = [int(o) for o in offs]
    return list(zip([0] + offs[:-1], offs))


def grouped_fwd(x_bits, w_bits, offs, mode=FLOOR):
    """Y[rows of group g] = mx_matmul(X[rows of g], W[g]); rows >= offs[-1] give zeros.

    x_bits [T, K], w_bits [E, N, K], offs = int32 inclusive cumulative group sizes
    (the `offs` argument of torch._grouped_mm at torchtitan/models/common/moe/moe.py:66-74).
    """
    T = x_bits.shape[0]
    E, N, K = w_bits.shape
    out = np.zeros((T, N), dtype=np.uint16)
    for g, (lo, hi) in enumerate(_group_bounds(offs)):
        if hi > lo:
            out[lo:hi] = mx_matmul(x_bits[lo:hi], w_bits[g], mode)
    return out


def grouped_dgrad(dy_bits, w_bits, offs, mode=FLOOR):
    """dX[rows of g] = deq(dY_g cast along N) @ deq(W_g cast along N)."""
    T = dy_bits.shape[0]
    E, N, K = w_bits.shape
    out = np.zeros((T, K), dtype=np.uint16)
    for g, (lo, hi) in enumerate(_group_bounds(offs)):
        if hi > lo:
            out[lo:hi] = linear_dgrad(dy_bits[lo:hi], w_bits[g], mode)
    return out


def grouped_wgrad(dy_bits, x_bits, offs, mode=FLOOR):
    """dW[g][N,K] = deq(dY_g cast along tokens)^T @ deq(X_g cast along tokens).

    Every group size must be a multiple of 32 so no block straddles a group boundary
    (torchtitan/models/common/moe/utils.py:47-52).  Empty groups give zeros.
    """
    N = dy_bits.shape[1]
    K = x_bits.shape[1]
    bounds = _group_bounds(offs)
    out = np.zeros((len(bounds), N, K), dtype=np.uint16)
    for g, (lo, hi) in enumerate(bounds):
        if (hi - lo) % BLOCK:
            raise ValueError("group sizes must be multiples of 32")
        if hi > lo:
            out[g] = linear_wgrad(dy_bits[lo:hi], x_bits[lo:hi], mode)
    return out


# --------------------------------------------------------------------------- scale layout
def scale_layout(scales: np.ndarray) -> np.ndarray:
    """Permute a [rows, nblk] scale matrix into the order the MFMA loop reads.

    Output is [ceil(rows/128), ceil(nblk/2), 64, 4] bytes: for row group rt, K step ks (64
    deep = 2 blocks), lane l and byte t the entry is scales[rt*128 + t*32 + (l & 31)][ks*2 + (l >> 5)],
    zero where that index is out of range.  One aligned dword per lane then holds the scales a
    32x32x64 MFMA lane needs for four consecutive 32-row sub-tiles.
    """
    rows, nblk = scales.shape
    rt_n = (rows + 127) // 128
    ks_n = (nblk + 1) // 2
    padded = np.zeros((rt_n * 128, ks_n * 2), dtype=np.uint8)
    padded[:rows, :nblk] = scales
    # [rt, t, i, ks, j] -> [rt, ks, j, i, t]
    v = padded.reshape(rt_n, 4, 32, ks_n, 2)
    return np.ascontiguousarray(v.transpose(0, 3, 4, 2, 1)).reshape(rt_n, ks_n, 64, 4)


def scale_unlayout(laid: np.ndarray, rows: int, nblk: int) -> np.ndarray:
    rt_n, ks_n = laid.shape[:2]
    v = laid.reshape(rt_n, ks_n, 2, 32, 4).transpose(0, 4, 3, 1, 2)
    return np.ascontiguousarray(v).reshape(rt_n * 128, ks_n * 2)[:rows, :nblk]


# --------------------------------------------------------------------------- group padding
def round_up(x: int, a: int) -> int:
    return (x + a - 1) // a * a


def generate_permute_indices(tokens_per_expert_group, experts_per_rank, num_ranks, max_len, alignment):
    """Index map from routed-token order to expert-grouped, alignment-padded order.

    Follows torchtitan/models/common/moe/kernels.py:145-218 (sizes/offsets) and :108-142
    (the fill): returns (permuted_indices int64 [max_len] with -1 in padding slots,
    m_sizes int32 [experts_per_rank], m_offsets int32 inclusive cumsum).
    """
    t = np.asarray(tokens_per_expert_group, dtype=np.int64)
    start = np.cumsum(t) - t
    total = t.reshape(num_ranks, -1).sum(0)
    total = np.maximum(total, alignment)
    m_sizes = ((total + alignment - 1) // alignment * alignment).astype(np.int32)
    m_offsets = np.cumsum(m_sizes.astype(np.int64))
    write = m_offsets - m_sizes
    perm = np.full(max_len, -1, dtype=np.int64)
    for e in range(experts_per_rank):
        ws = int(write[e])
        for r in range(num_ranks):
            i = r * experts_per_rank + e
            n = int(t[i])
            if n > 0:
                end = min(ws + n, max_len)
                if ws < end:
                    perm[ws:end] = np.arange(start[i], start[i] + (end - ws))
            ws += n
    return perm, m_sizes, m_offsets.astype(np.int32)


def padded_max_len(num_tokens: int, num_experts: int, alignment: int) -> int:
    """torchtitan/models/common/moe/utils.py:66-68."""
    return round_up(num_tokens + num_experts * alignment, alignment)


# --------------------------------------------------------------------------- inputs
def rms_norm_bf16(x_bits: np.ndarray, w_bits: np.ndarray, eps: float):
    """(y, rstd): y = bf16(w * (x * rstd)), rstd = 1 / sqrt(mean(x^2) + eps) per row, in float64
    from bf16 inputs (nn.RMSNorm with a weight, torchtitan/models/common/rmsnorm.py:14-50).
    A float32 reduction gives rstd to a few 1e-7 relative, which moves y to the neighbouring
    bf16 value at a few elements in a thousand: PARITY UNPINNED to that extent (tests bound it)."""
    x = bf16_bits_to_f32(x_bits).astype(np.float64)
    w = bf16_bits_to_f32(w_bits).astype(np.float64)
    rstd = 1.0 / np.sqrt((x * x).mean(axis=1) + eps)
    y = w[None, :] * (x * rstd[:, None])
    return f32_to_bf16_bits(y.astype(np.float32)), rstd


def silu_bf16(a_bits: np.ndarray) -> np.ndarray:
    """bf16 silu as one tensor op: x / (1 + exp(-x)) evaluated in float64 with float32's range
    (exp(-x) beyond float32 is infinite, so x below about -88.7 gives -0), rounded to bf16."""
    with np.errstate(over="ignore", invalid="ignore"):
        a = bf16_bits_to_f32(a_bits).astype(np.float64)
        e = np.exp(-a).astype(np.float32).astype(np.float64)
        s = a / (1.0 + e)
    return f32_to_bf16_bits(s.astype(np.float32))


def mul_bf16(x_bits: np.ndarray, y_bits: np.ndarray) -> np.ndarray:
    """bf16 product as one tensor op: exact in float32 (8 x 8 significand bits), rounded to bf16."""
    with np.errstate(over="ignore", invalid="ignore"):
        return f32_to_bf16_bits(bf16_bits_to_f32(x_bits) * bf16_bits_to_f32(y_bits))


def swiglu_bf16(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    """g = silu(a) * b as two bf16 tensor ops (torchtitan/models/common/feed_forward.py:61-62:
    ``F.silu(self.w1(x)) * self.w3(x)`` on bf16 activations).

    Pinning: the sigmoid is the textbook closed form in float64 and the product is exact before
    its rounding.  A float32 evaluation of silu with a library or hardware exp can land on the
    other side of a bf16 rounding boundary (the neighbouring bf16 value) for a few elements in
    ten thousand: PARITY UNPINNED to that extent, and the tests bound it to exactly that."""
    return mul_bf16(silu_bf16(a_bits), b_bits)


def swiglu_backward_bf16(dg_bits: np.ndarray, a_bits: np.ndarray, b_bits: np.ndarray):
    """(da, db) of g = silu(a) * b as bf16 autograd forms them (feed_forward.py:61-62 under
    autograd): the product node gives db = bf16(dg * silu_bf16(a)) and t = bf16(dg * b); the silu
    node gives da = bf16(t * s * (1 + a * (1 - s))), s = 1 / (1 + exp(-a)), evaluated here in
    float64 with float32's exp range.

    Pinning: db is exact given silu_bf16; da is the closed form of d silu / da (checked against
    a central difference and torch's CPU op in the tests); its last bf16 ulp under a float32
    evaluation is PARITY UNPINNED, as for silu_bf16."""
    db = mul_bf16(dg_bits, silu_bf16(a_bits))
    t = bf16_bits_to_f32(mul_bf16(dg_bits, b_bits)).astype(np.float64)
    with np.errstate(over="ignore", invalid="ignore"):
        a = bf16_bits_to_f32(a_bits).astype(np.float64)
        e = np.exp(-a).astype(np.float32).astype(np.float64)
        s = 1.0 / (1.0 + e)
        da = t * s * (1.0 + a * (1.0 - s))
        return f32_to_bf16_bits(da.astype(np.float32)), db


def moe_route_plan(counts: np.ndarray, order: np.ndarray, scores: np.ndarray | None, top_k: int,
                   alignment: int):
    """Aligned group layout of an MoE layer's routed pairs, composed from the padding rule of
    `generate_permute_indices` (moe/kernels.py:145-218) and the expert-sorted pair order
    (moe.py:355-362): (padded inclusive ends, token per padded row or -1, score per padded row,
    padded row per pair)."""
    E, R = len(counts), len(order)
    max_len = round_up(R + alignment * E, alignment)
    perm, _, m_offsets = generate_permute_indices(np.asarray(counts), E, 1, max_len, alignment)
    src_row = np.full(max_len, -1, dtype=np.int64)
    row_score = np.zeros(max_len, dtype=np.float32)
    pos = np.full(R, -1, dtype=np.int64)
    for p, i in enumerate(perm):
        if i >= 0:
            pair = order[i]
            src_row[p] = pair // top_k
            if scores is not None:
                row_score[p] = scores[pair]
            pos[pair] = p
    return m_offsets, src_row, row_score, pos


def gather_rows(x_bits: np.ndarray, row_index: np.ndarray, row_scale: np.ndarray | None = None) -> np.ndarray:
    """Rows x[row_index] with rows of zeros where the index is outside x (the -1 padding slots
    of torchtitan/models/common/moe/utils.py:78-80), optionally multiplied by a float32 score
    per row with the product rounded to bf16 (moe.py:521-527)."""
    n = x_bits.shape[0]
    ok = (row_index >= 0) & (row_index < n)
    rows = np.where(ok[:, None], x_bits[np.clip(row_index, 0, max(n - 1, 0))], 0).astype(np.uint16)
    if row_scale is None:
        return rows
    with np.errstate(over="ignore", invalid="ignore"):
        scaled = f32_to_bf16_bits(bf16_bits_to_f32(rows) * row_scale.astype(np.float32)[:, None])
    return np.where(ok[:, None], scaled, 0).astype(np.uint16)


def add_bf16(x_bits: np.ndarray, y_bits: np.ndarray) -> np.ndarray:
    """bf16 sum as one tensor op: float32 addition (exact for two bf16 operands up to its own
    rounding) rounded to bf16."""
    with np.errstate(over="ignore", invalid="ignore"):
        return f32_to_bf16_bits(bf16_bits_to_f32(x_bits) + bf16_bits_to_f32(y_bits))


def moe_combine(y_bits: np.ndarray, pos: np.ndarray, weights: np.ndarray | None = None) -> np.ndarray:
    """out[t] = sum_j weights[t, j] * y[pos[t, j]] accumulated in float32 for j = 0 .. k-1 in
    that order (product and sum rounded separately), rounded to bf16: the score-weighted
    combine of the top-k expert outputs (moe.py:535-555, where a scatter, a float upcast and a
    bmm / sum do it).  The reference's own summation order inside bmm / sum is not specified:
    PARITY UNPINNED in the last float32 bit of the accumulation; against an exact sum the result
    is within one bf16 step (tested)."""
    T, k = pos.shape
    y = bf16_bits_to_f32(y_bits)
    acc = np.zeros((T, y.shape[1]), dtype=np.float32)
    for j in range(k):
        r = pos[:, j]
        ok = (r >= 0) & (r < y.shape[0])
        rows = y[np.clip(r, 0, y.shape[0] - 1)]
        with np.errstate(over="ignore", invalid="ignore"):
            term = rows if weights is None else (weights[:, j].astype(np.float32)[:, None] * rows).astype(np.float32)
            acc = np.where(ok[:, None], (acc + term).astype(np.float32), acc)
    return f32_to_bf16_bits(acc)


def moe_row_dot(a_bits: np.ndarray, ia: np.ndarray, b_bits: np.ndarray, ib: np.ndarray) -> np.ndarray:
    """out[i] = <a[ia[i]], b[ib[i]]> in float64 (the gradient of a routing score is the dot
    product of the two rows its product joined); 0 where an index is outside its matrix."""
    a, b = bf16_bits_to_f32(a_bits).astype(np.float64), bf16_bits_to_f32(b_bits).astype(np.float64)
    ok = (ia >= 0) & (ia < a.shape[0]) & (ib >= 0) & (ib < b.shape[0])
    d = np.einsum("ij,ij->i", a[np.clip(ia, 0, a.shape[0] - 1)], b[np.clip(ib, 0, b.shape[0] - 1)])
    return np.where(ok, d, 0.0)


def token_log_probs(logits_bits: np.ndarray, target: np.ndarray):
    """(log-probability of target[r] under softmax(logits[r]), log-sum-exp per row) in float64
    from bf16 logits: what `.to(float32)`, `F.log_softmax` and `gather` compute in
    torchtitan/experiments/rl/unified/actors/utils.py:37-50."""
    x = bf16_bits_to_f32(logits_bits).astype(np.float64)
    m = x.max(axis=1, keepdims=True)
    lse = (m + np.log(np.exp(x - m).sum(axis=1, keepdims=True)))[:, 0]
    return x[np.arange(x.shape[0]), target] - lse, lse


def token_log_probs_grad(logits_bits: np.ndarray, target: np.ndarray, grad: np.ndarray) -> np.ndarray:
    """d/dlogits of sum_r grad[r] * logprob[r]: grad[r] * (onehot(target[r]) - softmax(x[r])), float64."""
    x = bf16_bits_to_f32(logits_bits).astype(np.float64)
    _, lse = token_log_probs(logits_bits, target)
    d = -np.exp(x - lse[:, None])
    d[np.arange(x.shape[0]), target] += 1.0
    return d * grad[:, None]


def policy_gradient_loss(policy_lps, ref_lps, advantages, kl_coef=0.1, ppo_clip_eps=0.2, entropy_coef=0.01):
    """GRPO / PPO loss of actors/utils.py:97-134 in float64 from per-sample token log-probs.
    Returns (total, dict of pg_loss, entropy, kl_div, ratio_mean, ratio_clipped_frac)."""
    mlr, mkl = [], []
    for p, r in zip(policy_lps, ref_lps):
        d = np.asarray(p, np.float64) - np.asarray(r, np.float64)
        mlr.append(d.mean())
        mkl.append((np.exp(d) - 1.0 - d).mean())
    ratio = np.exp(np.array(mlr))
    adv = np.asarray(advantages, np.float64)
    clipped = np.clip(ratio, 1 - ppo_clip_eps, 1 + ppo_clip_eps)
    pg = -np.minimum(ratio * adv, clipped * adv).mean()
    entropy = -np.concatenate([np.asarray(p, np.float64) for p in policy_lps]).mean()
    kl = float(np.mean(mkl))
    total = pg - entropy_coef * entropy + kl_coef * kl
    return total, {"pg_loss": pg, "entropy": entropy, "kl_div": kl, "ratio_mean": ratio.mean(),
                   "ratio_clipped_frac": float((np.abs(ratio - clipped) > 1e-6).mean())}


def make_cfg1_inputs(seed: int, M: int = 8192, K: int = 4096, N: int = 4096):
    """Seeded N(0,1) bf16 X[M,K], W[N,K] with 0.1 % of entries scaled by 100."""
    rng = np.random.default_rng(seed)

    def one(r, c):
        x = rng.standard_normal((r, c), dtype=np.float32)
        x = np.where(rng.random((r, c)) < 1e-3, x * np.float32(100.0), x)
        return f32_to_bf16_bits(x)

    return one(M, K), one(N, K)
