"""Tensor-level wrappers over the C ABI (include/mxfp8.h).

PyTorch is used for device memory and the current HIP stream only; every computation is a
call into libmxfp8_gfx950.so.  There is no fallback path: CPU tensors are rejected.
"""
from __future__ import annotations

import ctypes
import os
from typing import NamedTuple

import torch

from . import _lib
from ._lib import MX_SCALE_FLOOR, MX_SCALE_RCEIL, MX_SCALES_MFMA, MX_SCALES_ROWMAJOR

BLOCK = 32  # torchtitan/components/quantization/__init__.py:36

SCALE_MODES = {"floor": MX_SCALE_FLOOR, "rceil": MX_SCALE_RCEIL}


class MXData(NamedTuple):
    """e4m3 codes [rows, cols] (uint8) + E8M0 scales, blocks of 32 along `cols`."""

    codes: torch.Tensor
    scales: torch.Tensor
    scale_order: int  # MX_SCALES_ROWMAJOR: [rows, cols/32]; MX_SCALES_MFMA: flat re-laid buffer


class KernelTimer:
    """Optional per-launch timing with HIP events on the launch stream (used by bench.py).

    While a timer is installed with ``set_kernel_timer`` every library call is bracketed by two
    events recorded on the stream it is launched on; ``summary()`` synchronises once and
    returns {kernel name: (launches, mean milliseconds)}.
    """

    def __init__(self):
        self.records = []

    def bracket(self, name: str, device):
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        self.records.append((name, start, stop))
        return start, stop

    def summary(self):
        torch.cuda.synchronize()
        acc: dict[str, list[float]] = {}
        for name, a, b in self.records:
            acc.setdefault(name, []).append(a.elapsed_time(b))
        return {k: (len(v), sum(v) / len(v)) for k, v in acc.items()}


_timer: KernelTimer | None = None


def set_kernel_timer(timer: KernelTimer | None) -> None:
    global _timer
    _timer = timer


def _call(name: str, tag: str, device, *args) -> None:
    """Run one C-ABI entry point on `device`'s current stream and raise on a non-zero status."""
    fn = getattr(_lib.load(), name)
    with torch.cuda.device(device):
        if _timer is None:
            st = fn(*args)
        else:
            start, stop = _timer.bracket(tag, device)
            start.record()
            st = fn(*args)
            stop.record()
    _lib.check(st, name)


def _mode(mode) -> int:
    if isinstance(mode, str):
        return SCALE_MODES[mode]
    if mode not in (MX_SCALE_FLOOR, MX_SCALE_RCEIL):
        raise ValueError(f"unknown scale mode {mode!r}")
    return int(mode)


def _stream(t: torch.Tensor) -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _ptr(t: torch.Tensor) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr())


def _wrote(out: torch.Tensor) -> torch.Tensor:
    """A library write into a caller's tensor is an in-place op that autograd did not see: bump
    the version counter so that whatever is keyed on it (saved-tensor checks, the activation cast
    reuse of mx_tensor) notices the new contents."""
    torch.autograd.graph.increment_version(out)
    return out


def _check_hp(x: torch.Tensor) -> torch.Tensor:
    if not x.is_cuda:
        raise _lib.MXLibraryError("the MXFP8 kernels run on the GPU only; got a CPU tensor")
    if x.dtype != torch.bfloat16:
        raise TypeError(f"to_mx expects bfloat16, got {x.dtype}")
    if x.dim() != 2:
        raise ValueError("to_mx expects a 2-D tensor")
    if x.stride(1) != 1:
        x = x.contiguous()
    return x


def mfma_scale_bytes(rows: int, nblk: int) -> int:
    return ((rows + 127) // 128) * ((nblk + 1) // 2) * 256


def _alloc_scales(rows: int, nblk: int, order: int, device) -> torch.Tensor:
    if order == MX_SCALES_MFMA:
        return torch.empty(mfma_scale_bytes(rows, nblk), dtype=torch.uint8, device=device)
    return torch.empty((rows, nblk), dtype=torch.uint8, device=device)


def to_mx_dim0(x: torch.Tensor, mode="floor", order: int = MX_SCALES_ROWMAJOR) -> MXData:
    """Row-wise cast: blocks of 32 along the last dim of x [R, C]."""
    x = _check_hp(x)
    R, C = x.shape
    if C % BLOCK:
        raise ValueError(f"last dim {C} is not a multiple of {BLOCK}")
    codes = torch.empty((R, C), dtype=torch.uint8, device=x.device)
    scales = _alloc_scales(R, C // BLOCK, order, x.device)
    _call("mx_cast_dim0", "cast_dim0", x.device, _ptr(x), R, C, x.stride(0), _ptr(codes), _ptr(scales), _mode(mode), order, _stream(x))
    return MXData(codes, scales, order)


def to_mx_dim1(x: torch.Tensor, mode="floor", order: int = MX_SCALES_ROWMAJOR) -> MXData:
    """Column-wise cast of x [R, C]: codes [C, R], blocks of 32 down the rows of x."""
    x = _check_hp(x)
    R, C = x.shape
    if R % BLOCK:
        raise ValueError(f"first dim {R} is not a multiple of {BLOCK}")
    codes = torch.empty((C, R), dtype=torch.uint8, device=x.device)
    scales = _alloc_scales(C, R // BLOCK, order, x.device)
    _call("mx_cast_dim1", "cast_dim1", x.device, _ptr(x), R, C, x.stride(0), _ptr(codes), _ptr(scales), _mode(mode), order, _stream(x))
    return MXData(codes, scales, order)


# Row pitch of GEMM operands: codes whose rows lie a whole number of 4 KB apart (K = 4096, 14336,
# 16384 ...) put the lines a GEMM fetches together -- one 128-byte K block of 512 rows -- on few
# channels of the L2; 128 bytes between the end of a row and the start of the next spread them
# (measured on the dense GEMM inside the benchmark step: 2.4 % less time per launch).
# (MXFP8_CODE_PITCH_PAD in the environment: another multiple of 128, 0 = dense codes; for measurements.)
CODE_PITCH_PAD = int(os.environ.get("MXFP8_CODE_PITCH_PAD", "128"))


def _code_rows(rows: int, cols: int, pad: int, device, stack: int = 0) -> torch.Tensor:
    """uint8 [rows, cols] (or [stack, rows, cols]) whose rows lie cols + pad bytes apart."""
    shape = (rows, cols + pad) if not stack else (stack, rows, cols + pad)
    return torch.empty(shape, dtype=torch.uint8, device=device)[..., :cols]


def _pitch_ok(pad: int) -> int:
    """The row pitch padding the tile casts take: a multiple of 16 bytes (else none)."""
    return pad if pad > 0 and pad % 16 == 0 else 0


def to_mx_dim0_dim1(x: torch.Tensor, mode="floor", order: int = MX_SCALES_ROWMAJOR, pitch_pad: int = 0):
    """Both casts from one read of x; returns (row-wise MXData, column-wise MXData).  With
    `pitch_pad` the rows of both code matrices lie that many bytes further apart than they are
    long (`codes.stride(0)` says so; only `mx_gemm_nt` takes such operands), where the tile kernel
    takes the input; otherwise the codes are dense."""
    x = _check_hp(x)
    R, C = x.shape
    if R % BLOCK or C % BLOCK:
        raise ValueError(f"both dims of {tuple(x.shape)} must be multiples of {BLOCK}")
    scales = _alloc_scales(R, C // BLOCK, order, x.device)
    scales_t = _alloc_scales(C, R // BLOCK, order, x.device)
    if pitch_pad and pitch_pad % 16 == 0 and x.data_ptr() % 16 == 0 and C % 8 == 0 and x.stride(0) % 8 == 0:
        codes = torch.empty((R, C + pitch_pad), dtype=torch.uint8, device=x.device)[:, :C]
        codes_t = torch.empty((C, R + pitch_pad), dtype=torch.uint8, device=x.device)[:, :R]
        _call("mx_cast_dim0_dim1_ld", "cast_dim0_dim1", x.device, _ptr(x), R, C, x.stride(0), _ptr(codes),
              codes.stride(0), _ptr(scales), _ptr(codes_t), codes_t.stride(0), _ptr(scales_t), _mode(mode), order,
              _stream(x))
        return MXData(codes, scales, order), MXData(codes_t, scales_t, order)
    codes = torch.empty((R, C), dtype=torch.uint8, device=x.device)
    codes_t = torch.empty((C, R), dtype=torch.uint8, device=x.device)
    _call("mx_cast_dim0_dim1", "cast_dim0_dim1", x.device, _ptr(x), R, C, x.stride(0), _ptr(codes), _ptr(scales), _ptr(codes_t), _ptr(scales_t), _mode(mode), order, _stream(x))
    return MXData(codes, scales, order), MXData(codes_t, scales_t, order)


def to_mx_rows_gathered(x: torch.Tensor, row_index: torch.Tensor, mode="floor",
                        order: int = MX_SCALES_ROWMAJOR, want_cols: bool = True,
                        row_scale: torch.Tensor | None = None):
    """Casts of x[row_index] (index -1, or any index outside x, = a row of zeros) without forming
    the gathered tensor; returns (row-wise MXData, column-wise MXData or None).  `row_scale`
    (float32, one per output row) multiplies the rows in float32, rounded to bf16, first."""
    x = _check_hp(x)
    if row_scale is not None:
        if row_scale.dtype != torch.float32 or row_scale.shape != row_index.shape or row_scale.device != x.device:
            raise TypeError("row_scale must be float32 with one entry per output row on x's device")
        row_scale = row_scale.contiguous()
    if row_index.dtype != torch.int64 or row_index.dim() != 1 or row_index.device != x.device:
        raise TypeError("row_index must be a 1-D int64 tensor on x's device")
    row_index = row_index.contiguous()
    R, C = row_index.numel(), x.shape[1]
    if C % BLOCK or (want_cols and R % BLOCK):
        raise ValueError(f"dims {R}, {C} must be multiples of {BLOCK}")
    codes = torch.empty((R, C), dtype=torch.uint8, device=x.device)
    scales = _alloc_scales(R, C // BLOCK, order, x.device)
    codes_t = scales_t = None
    if want_cols:
        codes_t = torch.empty((C, R), dtype=torch.uint8, device=x.device)
        scales_t = _alloc_scales(C, R // BLOCK, order, x.device)
    _call("mx_cast_rows_gathered", "cast_rows_gathered", x.device, _ptr(x), _ptr(row_index),
          _ptr(row_scale) if row_scale is not None else None, x.shape[0],
          R, C, x.stride(0), _ptr(codes), _ptr(scales), _ptr(codes_t) if want_cols else None,
          _ptr(scales_t) if want_cols else None, _mode(mode), order, _stream(x))
    return MXData(codes, scales, order), (MXData(codes_t, scales_t, order) if want_cols else None)


def moe_route_plan(counts: torch.Tensor, order: torch.Tensor, scores: torch.Tensor | None, top_k: int,
                   alignment: int, length_multiple: int = 1):
    """(padded inclusive group ends int32 [E], token of every padded row int64 [max_len] (-1 =
    padding), score of every padded row float32 [max_len], padded row of every (token, choice)
    pair int64 [pairs]) for tokens-per-expert `counts` and the expert-sorted pair order; the
    padded length is the static bound round_up(pairs + alignment * E, alignment), rounded up
    further to `length_multiple` (a multiple of the alignment) when one is given."""
    if not counts.is_cuda:
        raise _lib.MXLibraryError("moe_route_plan runs on the GPU only")
    dev = counts.device
    c32 = counts.to(torch.int32).contiguous()
    E, R = c32.numel(), order.numel()
    if order.dtype != torch.int64 or order.device != dev:
        raise TypeError("order must be int64 on the counts' device")
    order = order.contiguous()
    if scores is not None:
        if scores.dtype != torch.float32 or scores.numel() != R or scores.device != dev:
            raise TypeError("scores must be float32 with one entry per pair")
        scores = scores.contiguous()
    step = max(alignment, length_multiple)
    if step % alignment:
        raise ValueError("length_multiple must be a multiple of the alignment")
    max_len = -(-(R + alignment * E) // step) * step
    offs = torch.empty(E, dtype=torch.int32, device=dev)
    src_row = torch.empty(max_len, dtype=torch.int64, device=dev)
    row_score = torch.empty(max_len, dtype=torch.float32, device=dev)
    pos = torch.full((R,), -1, dtype=torch.int64, device=dev)
    _call("mx_moe_route_plan", "moe_route_plan", dev, _ptr(c32), E, _ptr(order),
          _ptr(scores) if scores is not None else None, R, top_k, max_len, alignment, _ptr(offs),
          _ptr(src_row), _ptr(row_score), _ptr(pos), _stream(counts))
    return offs, src_row, row_score, pos


def moe_combine(y: torch.Tensor, pos: torch.Tensor, weights: torch.Tensor | None = None,
                y2: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = sum_j weights[t, j] * y[pos[t, j]] (float32, j in order; plain sum without
    weights), bf16 [tokens, cols].  y: bf16 [rows, cols]; pos: int64 [tokens, top_k]; a position
    outside y contributes nothing.  With y2 (y's shape) the rows are bf16(y + y2)."""
    y = _check_hp(y)
    if y2 is not None:
        y2 = _check_hp(y2)
        if y2.shape != y.shape or y2.stride(0) != y.stride(0):
            raise ValueError("y2 must have y's shape and row stride")
    if pos.dtype != torch.int64 or pos.dim() != 2 or pos.device != y.device:
        raise TypeError("pos must be a 2-D int64 tensor on y's device")
    pos = pos.contiguous()
    T, k = pos.shape
    if weights is not None:
        if weights.dtype != torch.float32 or weights.shape != pos.shape or weights.device != y.device:
            raise TypeError("weights must be float32 of pos's shape on y's device")
        weights = weights.contiguous()
    out = torch.empty((T, y.shape[1]), dtype=torch.bfloat16, device=y.device)
    _call("mx_moe_combine", "moe_combine", y.device, _ptr(y), _ptr(y2) if y2 is not None else None,
          y.shape[0], y.stride(0), _ptr(pos),
          _ptr(weights) if weights is not None else None, T, k, y.shape[1], _ptr(out), out.stride(0),
          _stream(y))
    return out


def moe_row_dot(a: torch.Tensor, ia: torch.Tensor, b: torch.Tensor, ib: torch.Tensor,
                a2: torch.Tensor | None = None) -> torch.Tensor:
    """out[i] = <a[ia[i]], b[ib[i]]> in float32 for bf16 matrices a, b with equal column counts;
    an index outside its matrix gives 0.  With a2 (a's shape) a's rows are bf16(a + a2)."""
    a, b = _check_hp(a), _check_hp(b)
    if a2 is not None:
        a2 = _check_hp(a2)
        if a2.shape != a.shape or a2.stride(0) != a.stride(0):
            raise ValueError("a2 must have a's shape and row stride")
    if a.shape[1] != b.shape[1]:
        raise ValueError(f"column mismatch: {a.shape[1]} vs {b.shape[1]}")
    for idx in (ia, ib):
        if idx.dtype != torch.int64 or idx.device != a.device:
            raise TypeError("indices must be int64 on the matrices' device")
    if ia.shape != ib.shape:
        raise ValueError("index shapes differ")
    ia_c, ib_c = ia.contiguous().view(-1), ib.contiguous().view(-1)
    out = torch.empty(ia.shape, dtype=torch.float32, device=a.device)
    _call("mx_moe_row_dot", "moe_row_dot", a.device, _ptr(a), _ptr(a2) if a2 is not None else None,
          a.shape[0], a.stride(0), _ptr(ia_c), _ptr(b),
          b.shape[0], b.stride(0), _ptr(ib_c), ia_c.numel(), a.shape[1], _ptr(out), _stream(a))
    return out


def mx_dequant(d: MXData, out: torch.Tensor | None = None) -> torch.Tensor:
    """bf16 [rows, cols] values of row-wise MXFP8 data (codes [rows, cols], blocks along cols)."""
    codes = d.codes
    if codes.dtype != torch.uint8 or codes.dim() != 2 or not codes.is_cuda:
        raise TypeError("expected 2-D uint8 codes on the GPU")
    codes = codes.contiguous()
    rows, cols = codes.shape
    if cols % BLOCK:
        raise ValueError(f"cols {cols} is not a multiple of {BLOCK}")
    if out is None:
        out = torch.empty((rows, cols), dtype=torch.bfloat16, device=codes.device)
    else:
        _wrote(out)
    scales = d.scales.contiguous()
    _call("mx_dequant", "dequant", codes.device, _ptr(codes), _ptr(scales), rows, cols, d.scale_order,
          _ptr(out), out.stride(0), _stream(codes))
    return out


def token_logprob_fwd(logits: torch.Tensor, target: torch.Tensor):
    """(log-probability of target[r] under softmax(logits[r]), log-sum-exp of row r), float32
    [rows], from bf16 logits [rows, vocab] read once."""
    logits = _check_hp(logits)
    if target.dtype != torch.int64 or target.shape != (logits.shape[0],) or target.device != logits.device:
        raise TypeError("target must be int64 [rows] on the logits' device")
    if logits.stride(0) % 8 or logits.data_ptr() % 16:
        logits = logits.contiguous().clone() if logits.shape[1] % 8 == 0 else _pad_row_stride(logits)
    target = target.contiguous()
    rows, vocab = logits.shape
    lp = torch.empty(rows, dtype=torch.float32, device=logits.device)
    lse = torch.empty(rows, dtype=torch.float32, device=logits.device)
    _call("mx_token_logprob_fwd", "token_logprob_fwd", logits.device, _ptr(logits), rows, vocab,
          logits.stride(0), _ptr(target), _ptr(lp), _ptr(lse), _stream(logits))
    return lp, lse


def _pad_row_stride(x: torch.Tensor) -> torch.Tensor:
    """Copy of x [rows, cols] whose row stride is a multiple of 8 elements (16-byte aligned rows)."""
    rows, cols = x.shape
    buf = torch.empty((rows, -(-cols // 8) * 8), dtype=x.dtype, device=x.device)
    view = buf[:, :cols]
    view.copy_(x)
    return view


def token_logprob_bwd(logits: torch.Tensor, target: torch.Tensor, lse: torch.Tensor,
                      grad_logprob: torch.Tensor) -> torch.Tensor:
    """Gradient of `token_logprob_fwd`'s first output with respect to the logits, bf16."""
    logits = _check_hp(logits)
    if logits.stride(0) % 8 or logits.data_ptr() % 16:
        logits = logits.contiguous().clone() if logits.shape[1] % 8 == 0 else _pad_row_stride(logits)
    rows, vocab = logits.shape
    g = grad_logprob.to(torch.float32).contiguous()
    lse, target = lse.contiguous(), target.contiguous()
    out = torch.empty((rows, -(-vocab // 8) * 8), dtype=torch.bfloat16, device=logits.device)[:, :vocab]
    step = 65535
    for lo in range(0, rows, step):
        n = min(step, rows - lo)
        _call("mx_token_logprob_bwd", "token_logprob_bwd", logits.device, _ptr(logits[lo:]), n, vocab,
              logits.stride(0), _ptr(target[lo:]), _ptr(lse[lo:]), _ptr(g[lo:]), _ptr(out[lo:]),
              out.stride(0), _stream(logits))
    return out


def rms_norm_to_mx(x: torch.Tensor, weight: torch.Tensor, eps: float, mode="floor",
                   order: int = MX_SCALES_ROWMAJOR, want_y: bool = False, pitch_pad: int = 0):
    """Both casts of y = rms_norm(x) * weight (float32 arithmetic, one rounding to bf16) without
    y passing through memory; returns (row-wise MXData, column-wise MXData, rstd float32 [rows],
    y or None).  `pitch_pad`: as for `to_mx_dim0_dim1`."""
    x = _check_hp(x)
    if weight.dtype != torch.bfloat16 or weight.shape != (x.shape[1],) or weight.device != x.device:
        raise TypeError("the norm weight must be bf16 [cols] on x's device")
    weight = weight.contiguous()
    R, C = x.shape
    if R % BLOCK or C % BLOCK:
        raise ValueError(f"both dims of {tuple(x.shape)} must be multiples of {BLOCK}")
    pad = _pitch_ok(pitch_pad)
    codes = _code_rows(R, C, pad, x.device)
    scales = _alloc_scales(R, C // BLOCK, order, x.device)
    codes_t = _code_rows(C, R, pad, x.device)
    scales_t = _alloc_scales(C, R // BLOCK, order, x.device)
    rstd = torch.empty(R, dtype=torch.float32, device=x.device)
    y = torch.empty((R, C), dtype=torch.bfloat16, device=x.device) if want_y else None
    _call("mx_rmsnorm_cast_dim0_dim1_ld", "rmsnorm_cast_dim0_dim1", x.device, _ptr(x), _ptr(weight),
          ctypes.c_float(eps), R, C, x.stride(0), _ptr(rstd), _ptr(y) if y is not None else None,
          _ptr(codes), codes.stride(0), _ptr(scales), _ptr(codes_t), codes_t.stride(0), _ptr(scales_t),
          _mode(mode), order, _stream(x))
    return MXData(codes, scales, order), MXData(codes_t, scales_t, order), rstd, y


def swiglu_to_mx_dim0_dim1(a: torch.Tensor, b: torch.Tensor, mode="floor",
                           order: int = MX_SCALES_ROWMAJOR, want_g: bool = False, pitch_pad: int = 0):
    """Both casts of g = silu(a) * b (bf16, every step rounded to bf16) without g passing through
    memory; returns (row-wise MXData, column-wise MXData, g or None).  `pitch_pad`: as for
    `to_mx_dim0_dim1`."""
    a, b = _check_hp(a), _check_hp(b)
    if a.shape != b.shape:
        raise ValueError(f"shape mismatch: {tuple(a.shape)} vs {tuple(b.shape)}")
    R, C = a.shape
    if R % BLOCK or C % BLOCK:
        raise ValueError(f"both dims of {tuple(a.shape)} must be multiples of {BLOCK}")
    pad = _pitch_ok(pitch_pad)
    codes = _code_rows(R, C, pad, a.device)
    scales = _alloc_scales(R, C // BLOCK, order, a.device)
    codes_t = _code_rows(C, R, pad, a.device)
    scales_t = _alloc_scales(C, R // BLOCK, order, a.device)
    g = torch.empty((R, C), dtype=torch.bfloat16, device=a.device) if want_g else None
    _call("mx_swiglu_cast_dim0_dim1_ld", "swiglu_cast_dim0_dim1", a.device, _ptr(a), _ptr(b), R, C,
          a.stride(0), b.stride(0), _ptr(codes), codes.stride(0), _ptr(scales), _ptr(codes_t), codes_t.stride(0),
          _ptr(scales_t), _ptr(g) if g is not None else None, _mode(mode), order, _stream(a))
    return MXData(codes, scales, order), MXData(codes_t, scales_t, order), g


def _scale_count(rows: int, nblk: int, order: int) -> int:
    return mfma_scale_bytes(rows, nblk) if order == MX_SCALES_MFMA else rows * nblk


def swiglu_bwd_to_mx_dim0_dim1(dg: torch.Tensor, a: torch.Tensor, b: torch.Tensor, mode="floor",
                               order: int = MX_SCALES_ROWMAJOR, want_grads: bool = False, pitch_pad: int = 0):
    """Backward of g = silu(a) * b with both casts of each gradient from one pass over dg, a, b.

    Returns ((da row-wise, da column-wise), (db row-wise, db column-wise), stacked bf16 [2, R, C]
    gradients or None).  The two row-wise (column-wise) results are the halves of one buffer.
    `pitch_pad`: as for `to_mx_dim0_dim1`."""
    dg, a, b = _check_hp(dg), _check_hp(a), _check_hp(b)
    if a.shape != b.shape or a.shape != dg.shape:
        raise ValueError(f"shape mismatch: {tuple(dg.shape)}, {tuple(a.shape)}, {tuple(b.shape)}")
    R, C = a.shape
    if R % BLOCK or C % BLOCK:
        raise ValueError(f"both dims of {tuple(a.shape)} must be multiples of {BLOCK}")
    dev = a.device
    n_s, n_st = _scale_count(R, C // BLOCK, order), _scale_count(C, R // BLOCK, order)
    pad = _pitch_ok(pitch_pad)
    codes = _code_rows(R, C, pad, dev, stack=2)
    codes_t = _code_rows(C, R, pad, dev, stack=2)
    scales = torch.empty(2 * n_s, dtype=torch.uint8, device=dev)
    scales_t = torch.empty(2 * n_st, dtype=torch.uint8, device=dev)
    dab = torch.empty((2, R, C), dtype=torch.bfloat16, device=dev) if want_grads else None
    _call("mx_swiglu_bwd_cast_dim0_dim1_ld", "swiglu_bwd_cast_dim0_dim1", dev, _ptr(dg), _ptr(a), _ptr(b),
          R, C, dg.stride(0), a.stride(0), b.stride(0), _ptr(codes), codes.stride(1), _ptr(scales), _ptr(codes_t),
          codes_t.stride(1), _ptr(scales_t), _ptr(dab) if dab is not None else None, _mode(mode), order, _stream(a))

    def half(i):
        s, st = scales[i * n_s:(i + 1) * n_s], scales_t[i * n_st:(i + 1) * n_st]
        if order == MX_SCALES_ROWMAJOR:
            s, st = s.view(R, C // BLOCK), st.view(C, R // BLOCK)
        return MXData(codes[i], s, order), MXData(codes_t[i], st, order)

    return half(0), half(1), dab


def scale_layout(scales: torch.Tensor) -> torch.Tensor:
    """Row-major [rows, nblk] scales -> flat buffer in MFMA order."""
    rows, nblk = scales.shape
    scales = scales.contiguous()
    out = torch.empty(mfma_scale_bytes(rows, nblk), dtype=torch.uint8, device=scales.device)
    _call("mx_scale_layout", "scale_layout", scales.device, _ptr(scales), rows, nblk, _ptr(out), _stream(scales))
    return out


def scale_unlayout(laid: torch.Tensor, rows: int, nblk: int) -> torch.Tensor:
    out = torch.empty((rows, nblk), dtype=torch.uint8, device=laid.device)
    _call("mx_scale_unlayout", "scale_unlayout", laid.device, _ptr(laid), rows, nblk, _ptr(out), _stream(laid))
    return out


def _as_mfma(d: MXData) -> torch.Tensor:
    return d.scales if d.scale_order == MX_SCALES_MFMA else scale_layout(d.scales)


_gemm_workspace: dict = {}  # (device index, M, N, K) -> bytes the library would split with


def _common_pitch(*codes, multiple: int = 128):
    """(the code matrices as the kernels take them, bytes between their rows): unit inner stride
    and one row pitch for all of them, a multiple of `multiple` where it is not the row length
    (copies are made where they differ)."""
    pitch = codes[0].stride(0)
    K = codes[0].shape[1]
    if any(c.stride(1) != 1 or c.stride(0) != pitch for c in codes) or (pitch != K and pitch % multiple):
        codes = tuple(c.contiguous() for c in codes)
        pitch = K
    return codes, pitch


def _gemm_nt_into(a_codes, a_scales, b_codes, b_scales, out):
    M, K = a_codes.shape
    N = b_codes.shape[0]
    (a_codes, b_codes), ldk = _common_pitch(a_codes, b_codes, multiple=16)  # (the tile kernels take any such pitch)
    key = (out.device.index, M, N, K)
    need = _gemm_workspace.get(key)
    if need is None:
        with torch.cuda.device(out.device):
            need = _gemm_workspace[key] = int(_lib.load().mx_gemm_nt_workspace_bytes(M, N, K))
    ws = None
    if need:  # few output tiles, long contraction: split over the CUs through float32 partial sums
        ws = torch.empty(need, dtype=torch.uint8, device=out.device)
    if ldk != K:
        _call("mx_gemm_nt_ld", "gemm_nt_splitk" if need else "gemm_nt", out.device, _ptr(a_codes), _ptr(a_scales),
              _ptr(b_codes), _ptr(b_scales), _ptr(out), M, N, K, ldk, out.stride(0),
              _ptr(ws) if need else None, need, _stream(out))
        return out
    if need:
        _call("mx_gemm_nt_ws", "gemm_nt_splitk", out.device, _ptr(a_codes), _ptr(a_scales), _ptr(b_codes),
              _ptr(b_scales), _ptr(out), M, N, K, out.stride(0), _ptr(ws), need, _stream(out))
        return out
    _call("mx_gemm_nt", "gemm_nt", out.device, _ptr(a_codes), _ptr(a_scales), _ptr(b_codes),
          _ptr(b_scales), _ptr(out), M, N, K, out.stride(0), _stream(out))
    return out


def _gemm_nt_op(a_codes, a_scales, b_codes, b_scales):
    out = torch.empty((a_codes.shape[0], b_codes.shape[0]), dtype=torch.bfloat16, device=a_codes.device)
    return _gemm_nt_into(a_codes, a_scales, b_codes, b_scales, out)


def _grouped_2d3d_into(a_codes, a_scales, a_order, b_codes, b_scales, offs, out):
    T, K = a_codes.shape
    G, N, _ = b_codes.shape
    _call("mx_grouped_gemm_2d3d", "grouped_gemm_2d3d", out.device, _ptr(a_codes), _ptr(a_scales),
          _ptr(b_codes), _ptr(b_scales), _ptr(offs), _ptr(out), T, N, K, G, out.stride(0), a_order,
          _stream(out))
    return out


def _grouped_2d3d_op(a_codes, a_scales, a_order, b_codes, b_scales, offs):
    out = torch.empty((a_codes.shape[0], b_codes.shape[1]), dtype=torch.bfloat16, device=a_codes.device)
    return _grouped_2d3d_into(a_codes, a_scales, a_order, b_codes, b_scales, offs, out)


def _grouped_2d3d_rows_out_op(a_codes, a_scales, b_codes, b_scales, offs, out_offs, out_rows, second=None):
    T, K = a_codes.shape
    G, N, _ = b_codes.shape
    out = torch.empty((out_rows, N), dtype=torch.bfloat16, device=a_codes.device)
    extra = [_ptr(t) for t in second] if second is not None else [None] * 4
    _call("mx_grouped_gemm_2d3d_rows_out", "grouped_gemm_2d3d_rows_out", out.device, _ptr(a_codes), _ptr(a_scales),
          _ptr(b_codes), _ptr(b_scales), *extra, _ptr(offs), _ptr(out_offs), _ptr(out), T, out_rows, N, K, G, N,
          _stream(out))
    return out


# The GEMMs whose output a forward pass hands on are also registered with torch's dispatcher, so
# that a per-op activation-checkpoint policy (torch.utils.checkpoint's selective contexts, which
# watch dispatched ops) can name them and keep their outputs instead of running them again in
# the recomputation.  The registered form is only taken while some dispatch mode is active; the
# plain eager path keeps calling the library directly.
_dispatcher_ops = torch.library.Library("torchtitan_amd", "DEF")
_dispatcher_ops.define("mx_gemm_nt(Tensor a_codes, Tensor a_scales, Tensor b_codes, Tensor b_scales) -> Tensor")
_dispatcher_ops.define("mx_grouped_gemm_2d3d(Tensor a_codes, Tensor a_scales, int a_order, Tensor b_codes, "
                       "Tensor b_scales, Tensor offs) -> Tensor")
_dispatcher_ops.define("mx_grouped_gemm_2d3d_rows_out(Tensor a_codes, Tensor a_scales, Tensor b_codes, "
                       "Tensor b_scales, Tensor offs, Tensor out_offs, int out_rows) -> Tensor")
_dispatcher_ops.impl("mx_gemm_nt", _gemm_nt_op, "CUDA")
_dispatcher_ops.impl("mx_grouped_gemm_2d3d", _grouped_2d3d_op, "CUDA")
_dispatcher_ops.impl("mx_grouped_gemm_2d3d_rows_out", _grouped_2d3d_rows_out_op, "CUDA")


_dispatch_depth = getattr(torch._C, "_len_torch_dispatch_stack", None)


def _watched() -> bool:
    """True while some TorchDispatchMode is active (a selective-checkpoint context is one)."""
    return _dispatch_depth is not None and _dispatch_depth() > 0


def op_sac_save_list() -> set:
    """The dispatcher ops of this package whose outputs a per-op activation-checkpoint policy may
    save (the forward GEMMs): add them to the model's save list
    (torchtitan/models/llama3/parallelize.py:44-60) to keep MXFP8 GEMM outputs through the
    recomputation, as the bf16 path keeps its `aten.mm` outputs.  Casts stay recomputed."""
    return {torch.ops.torchtitan_amd.mx_gemm_nt.default,
            torch.ops.torchtitan_amd.mx_grouped_gemm_2d3d.default,
            torch.ops.torchtitan_amd.mx_grouped_gemm_2d3d_rows_out.default}


def mx_gemm_nt(a: MXData, b: MXData, out: torch.Tensor | None = None) -> torch.Tensor:
    """bf16 D[M,N] = deq(a)[M,K] @ deq(b)[N,K]^T with fp32 accumulation."""
    M, K = a.codes.shape
    N, Kb = b.codes.shape
    if K != Kb:
        raise ValueError(f"contraction mismatch: {K} vs {Kb}")
    sa, sb = _as_mfma(a), _as_mfma(b)
    if out is None:
        if _watched():
            return torch.ops.torchtitan_amd.mx_gemm_nt(a.codes, sa, b.codes, sb)
        return _gemm_nt_op(a.codes, sa, b.codes, sb)
    if out.shape != (M, N) or out.dtype != torch.bfloat16 or out.stride(1) != 1:
        raise ValueError("out must be a bf16 [M, N] tensor with unit inner stride")
    return _gemm_nt_into(a.codes, sa, b.codes, sb, _wrote(out))


def mx_gemm_nt_pair(a: MXData, b: MXData, a2: MXData, b2: MXData) -> torch.Tensor:
    """bf16 deq(a) @ deq(b)^T + deq(a2) @ deq(b2)^T: one GEMM whose output tiles accumulate both
    products before they are rounded and written, where the persistent kernel takes the shape;
    otherwise two GEMMs and a bf16 add."""
    M, K = a.codes.shape
    N = b.codes.shape[0]
    if a2.codes.shape != (M, K) or b2.codes.shape != (N, K) or b.codes.shape[1] != K:
        raise ValueError("both operand sets must have the same shapes")
    if M <= 128 or N <= 128 or K % 128 or N % 8:
        return mx_gemm_nt(a, b) + mx_gemm_nt(a2, b2)
    out = torch.empty((M, N), dtype=torch.bfloat16, device=a.codes.device)
    sa, sb, sa2, sb2 = _as_mfma(a), _as_mfma(b), _as_mfma(a2), _as_mfma(b2)  # kept alive over the launch
    (ac, bc, a2c, b2c), ldk = _common_pitch(a.codes, b.codes, a2.codes, b2.codes)
    _call("mx_gemm_nt_pair_ld", "gemm_nt_pair", out.device, _ptr(ac), _ptr(sa), _ptr(bc), _ptr(sb),
          _ptr(a2c), _ptr(sa2), _ptr(b2c), _ptr(sb2), _ptr(out), M, N, K, ldk, N, _stream(out))
    return out


def _persistent_shape(M: int, N: int, K: int) -> bool:
    return M > 128 and N > 128 and K % 128 == 0 and N % 8 == 0


def mx_gemm_nt_shared_a(a: MXData, b: MXData, b2: MXData) -> torch.Tensor:
    """bf16 [2, M, N]: deq(a) @ deq(b)^T and deq(a) @ deq(b2)^T.  One launch in which the panels
    of `a` are fetched once for both products where the persistent kernel takes the shape,
    otherwise two GEMMs; bit-identical either way."""
    M, K = a.codes.shape
    N = b.codes.shape[0]
    if b2.codes.shape != b.codes.shape or b.codes.shape[1] != K:
        raise ValueError("both second operands must have the same shape")
    if _watched():  # as dispatcher ops, so that a per-op checkpoint policy can keep the outputs
        return torch.stack((mx_gemm_nt(a, b), mx_gemm_nt(a, b2)))
    out = torch.empty((2, M, N), dtype=torch.bfloat16, device=a.codes.device)
    if not _persistent_shape(M, N, K):
        mx_gemm_nt(a, b, out[0])
        mx_gemm_nt(a, b2, out[1])
        return out
    sa, sb, sb2 = _as_mfma(a), _as_mfma(b), _as_mfma(b2)
    (ac, bc, b2c), ldk = _common_pitch(a.codes, b.codes, b2.codes)
    _call("mx_gemm_nt_shared_a_ld", "gemm_nt_shared_a", out.device, _ptr(ac), _ptr(sa), _ptr(bc), _ptr(sb),
          _ptr(b2c), _ptr(sb2), _ptr(out[0]), _ptr(out[1]), M, N, K, ldk, N, _stream(out))
    return out


def mx_gemm_nt_shared_b(a: MXData, a2: MXData, b: MXData) -> torch.Tensor:
    """bf16 [2, M, N]: deq(a) @ deq(b)^T and deq(a2) @ deq(b)^T, as `mx_gemm_nt_shared_a` with the
    roles of the operands swapped."""
    M, K = a.codes.shape
    N = b.codes.shape[0]
    if a2.codes.shape != a.codes.shape or b.codes.shape[1] != K:
        raise ValueError("both first operands must have the same shape")
    out = torch.empty((2, M, N), dtype=torch.bfloat16, device=a.codes.device)
    if not _persistent_shape(M, N, K):
        mx_gemm_nt(a, b, out[0])
        mx_gemm_nt(a2, b, out[1])
        return out
    sa, sa2, sb = _as_mfma(a), _as_mfma(a2), _as_mfma(b)
    (ac, a2c, bc), ldk = _common_pitch(a.codes, a2.codes, b.codes)
    _call("mx_gemm_nt_shared_b_ld", "gemm_nt_shared_b", out.device, _ptr(ac), _ptr(sa), _ptr(a2c), _ptr(sa2),
          _ptr(bc), _ptr(sb), _ptr(out[0]), _ptr(out[1]), M, N, K, ldk, N, _stream(out))
    return out


# --------------------------------------------------------------------------- 3-D weights
def to_mx_dim0_batched(w: torch.Tensor, mode="floor", order: int = MX_SCALES_MFMA) -> MXData:
    """Row-wise cast of every matrix of w [G, R, C]: codes [G, R, C], one scale block each.

    A 3-D weight is G stacked matrices, so this is one row-wise cast of the [G*R, C] view; in
    MFMA order that equals G per-matrix blocks only when R is a multiple of 128, otherwise the
    matrices are cast one by one.
    """
    G, R, C = w.shape
    if order == MX_SCALES_MFMA and R % 128:
        parts = [to_mx_dim0(w[g], mode, order) for g in range(G)]
        return MXData(torch.stack([p.codes for p in parts]), torch.cat([p.scales for p in parts]), order)
    d = to_mx_dim0(w.reshape(G * R, C), mode, order)
    scales = d.scales if order == MX_SCALES_MFMA else d.scales.view(G, R, C // BLOCK)
    return MXData(d.codes.view(G, R, C), scales, order)


def to_mx_dim1_batched(w: torch.Tensor, mode="floor", order: int = MX_SCALES_MFMA) -> MXData:
    """Column-wise cast of every matrix of w [G, R, C]: codes [G, C, R]."""
    if w.dim() != 3 or w.dtype != torch.bfloat16 or not w.is_cuda:
        raise TypeError("expected a 3-D bf16 GPU tensor")
    w = w.contiguous()
    G, R, C = w.shape
    if R % BLOCK:
        raise ValueError(f"dim 1 ({R}) is not a multiple of {BLOCK}")
    codes = torch.empty((G, C, R), dtype=torch.uint8, device=w.device)
    per = mfma_scale_bytes(C, R // BLOCK) if order == MX_SCALES_MFMA else C * (R // BLOCK)
    scales = torch.empty(G * per, dtype=torch.uint8, device=w.device)
    _call("mx_cast_dim1_batched", "cast_dim1_batched", w.device, _ptr(w), G, R, C, C, _ptr(codes), _ptr(scales), _mode(mode), order, _stream(w))
    if order == MX_SCALES_ROWMAJOR:
        scales = scales.view(G, C, R // BLOCK)
    return MXData(codes, scales, order)


def to_mx_dim0_dim1_batched(w: torch.Tensor, mode="floor", order: int = MX_SCALES_MFMA):
    """Both casts of every matrix of w [G, R, C] from one read."""
    if w.dim() != 3 or w.dtype != torch.bfloat16 or not w.is_cuda:
        raise TypeError("expected a 3-D bf16 GPU tensor")
    w = w.contiguous()
    G, R, C = w.shape
    if R % BLOCK or C % BLOCK:
        raise ValueError(f"dims {R}, {C} must be multiples of {BLOCK}")
    codes = torch.empty((G, R, C), dtype=torch.uint8, device=w.device)
    codes_t = torch.empty((G, C, R), dtype=torch.uint8, device=w.device)
    if order == MX_SCALES_MFMA:
        per, per_t = mfma_scale_bytes(R, C // BLOCK), mfma_scale_bytes(C, R // BLOCK)
    else:
        per, per_t = R * (C // BLOCK), C * (R // BLOCK)
    scales = torch.empty(G * per, dtype=torch.uint8, device=w.device)
    scales_t = torch.empty(G * per_t, dtype=torch.uint8, device=w.device)
    _call("mx_cast_dim0_dim1_batched", "cast_dim0_dim1_batched", w.device, _ptr(w), G, R, C, C, _ptr(codes), _ptr(scales), _ptr(codes_t), _ptr(scales_t), _mode(mode), order, _stream(w))
    if order == MX_SCALES_ROWMAJOR:
        scales, scales_t = scales.view(G, R, C // BLOCK), scales_t.view(G, C, R // BLOCK)
    return MXData(codes, scales, order), MXData(codes_t, scales_t, order)


# --------------------------------------------------------------------------- grouped GEMMs
FAST_MAX_GROUPS = 510   # groups the persistent kernel keeps a table of in LDS
FAST_LENGTH_MULTIPLE = 128  # its operands' token axis: whole 128-deep K blocks / 128-row scale groups


def mx_grouped_gemm_2d3d(a: MXData, b: MXData, offs: torch.Tensor,
                         out: torch.Tensor | None = None) -> torch.Tensor:
    """out[rows of group g] = deq(a[rows of g]) @ deq(b[g])^T; rows past offs[-1] are zero.

    a: codes [T, K]; b: codes [G, N, K] with MFMA-order scales (G per-matrix blocks); offs:
    int32 [G] inclusive cumulative group sizes on the device.  With row-major scales for a the
    groups may end anywhere; with MFMA-order scales for a every group must end at a multiple
    of 32 rows (checked on the device: a violation fills the output with NaN) and the
    persistent kernel (csrc/mx_gemm32.hip) runs.
    """
    T, K = a.codes.shape
    G, N, Kb = b.codes.shape
    if K != Kb:
        raise ValueError(f"contraction mismatch: {K} vs {Kb}")
    if b.scale_order != MX_SCALES_MFMA:
        raise ValueError("2d3d expects MFMA-order scales for b")
    if offs.dtype != torch.int32 or offs.numel() != G:
        raise ValueError("offs must be int32 with one entry per group")
    if out is None:
        if _watched():
            return torch.ops.torchtitan_amd.mx_grouped_gemm_2d3d(a.codes, a.scales, a.scale_order,
                                                                 b.codes, b.scales, offs)
        return _grouped_2d3d_op(a.codes, a.scales, a.scale_order, b.codes, b.scales, offs)
    return _grouped_2d3d_into(a.codes, a.scales, a.scale_order, b.codes, b.scales, offs, _wrote(out))


def mx_grouped_gemm_2d3d_pair(a: MXData, b: MXData, a2: MXData, b2: MXData, offs: torch.Tensor,
                              out: torch.Tensor | None = None) -> torch.Tensor:
    """out[rows of g] = deq(a[rows of g]) @ deq(b[g])^T + deq(a2[rows of g]) @ deq(b2[g])^T, both
    sets with MFMA-order scales and 32-aligned groups (the persistent kernel); other layouts:
    two grouped GEMMs and a bf16 add."""
    T, K = a.codes.shape
    G, N, _ = b.codes.shape
    if a2.codes.shape != a.codes.shape or b2.codes.shape != b.codes.shape:
        raise ValueError("both operand sets must have the same shapes")
    fast = all(d.scale_order == MX_SCALES_MFMA for d in (a, b, a2, b2))
    if not fast or K % 128 or N % 8 or T % 32 or G > FAST_MAX_GROUPS:
        both = mx_grouped_gemm_2d3d(a, b, offs) + mx_grouped_gemm_2d3d(a2, b2, offs)
        return both if out is None else out.copy_(both)
    if offs.dtype != torch.int32 or offs.numel() != G:
        raise ValueError("offs must be int32 with one entry per group")
    if out is None:
        out = torch.empty((T, N), dtype=torch.bfloat16, device=a.codes.device)
    else:
        _wrote(out)
    _call("mx_grouped_gemm_2d3d_pair", "grouped_gemm_2d3d_pair", out.device, _ptr(a.codes), _ptr(a.scales),
          _ptr(b.codes), _ptr(b.scales), _ptr(a2.codes), _ptr(a2.scales), _ptr(b2.codes), _ptr(b2.scales),
          _ptr(offs), _ptr(out), T, N, K, G, out.stride(0), _stream(out))
    return out


def mx_grouped_gemm_2d3d_rows_out(a: MXData, b: MXData, offs: torch.Tensor, out_offs: torch.Tensor,
                                  out_rows: int, a2: MXData | None = None,
                                  b2: MXData | None = None) -> torch.Tensor:
    """bf16 [out_rows, N]: the grouped product (with a2, b2: the sum of two, as
    `mx_grouped_gemm_2d3d_pair`) of operands whose groups are padded, written without the padding:
    the first out_offs[g] - out_offs[g-1] rows of group g go to rows [out_offs[g-1], out_offs[g])
    (out_offs: int32 [G] inclusive ends on the device), rows from out_offs[-1] on are zero.

    Takes the place of the grouped GEMM followed by a gather of the unpadded rows (the second
    half of the padding wrapper, torchtitan/models/common/moe/utils.py:85-89 and :116).  MFMA-order scales and 32-aligned
    padded groups only (the persistent kernel); `rows_out_supported` tells.  The zero rows need
    a.codes to have at least as many rows behind its last group as the output has."""
    T, K = a.codes.shape
    G, N, _ = b.codes.shape
    if not rows_out_supported(a, b, a2, b2):
        raise ValueError("unpadded output needs MFMA-order scales, K % 128 == 0, N % 8 == 0, T % 32 == 0")
    for o in (offs, out_offs):
        if o.dtype != torch.int32 or o.numel() != G:
            raise ValueError("offs and out_offs must be int32 with one entry per group")
    if not 0 <= out_rows <= T:
        raise ValueError("the output cannot have more rows than the padded operand")
    if a2 is None:
        if _watched():  # as a dispatcher op: a forward GEMM whose output a checkpoint policy may keep
            return torch.ops.torchtitan_amd.mx_grouped_gemm_2d3d_rows_out(a.codes, a.scales, b.codes, b.scales,
                                                                          offs, out_offs, out_rows)
        return _grouped_2d3d_rows_out_op(a.codes, a.scales, b.codes, b.scales, offs, out_offs, out_rows)
    if a2.codes.shape != a.codes.shape or b2.codes.shape != b.codes.shape:
        raise ValueError("both operand sets must have the same shapes")
    return _grouped_2d3d_rows_out_op(a.codes, a.scales, b.codes, b.scales, offs, out_offs, out_rows,
                                     (a2.codes, a2.scales, b2.codes, b2.scales))


def rows_out_supported(a: MXData, b: MXData, a2: MXData | None = None, b2: MXData | None = None) -> bool:
    T, K = a.codes.shape
    G, N, _ = b.codes.shape
    every = [d for d in (a, b, a2, b2) if d is not None]
    return (len(every) in (2, 4) and all(d.scale_order == MX_SCALES_MFMA for d in every)
            and K % 128 == 0 and N % 8 == 0 and T % 32 == 0 and G <= FAST_MAX_GROUPS)


def mx_grouped_gemm_2d3d_shared_a(a: MXData, b: MXData, b2: MXData, offs: torch.Tensor) -> torch.Tensor:
    """bf16 [2, T, N]: grouped a x b[g]^T and grouped a x b2[g]^T.  One launch of the persistent
    kernel over both products when every scale buffer is in MFMA order (32-aligned groups),
    otherwise two grouped GEMMs; bit-identical either way."""
    T, K = a.codes.shape
    G, N, _ = b.codes.shape
    if b2.codes.shape != b.codes.shape:
        raise ValueError("both weight stacks must have the same shape")
    if offs.dtype != torch.int32 or offs.numel() != G:
        raise ValueError("offs must be int32 with one entry per group")
    if _watched():  # as dispatcher ops, so that a per-op checkpoint policy can keep the outputs
        return torch.stack((mx_grouped_gemm_2d3d(a, b, offs), mx_grouped_gemm_2d3d(a, b2, offs)))
    out = torch.empty((2, T, N), dtype=torch.bfloat16, device=a.codes.device)
    fast = all(d.scale_order == MX_SCALES_MFMA for d in (a, b, b2))
    if not fast or K % 128 or N % 8 or T % 32 or G > FAST_MAX_GROUPS:
        mx_grouped_gemm_2d3d(a, b, offs, out[0])
        mx_grouped_gemm_2d3d(a, b2, offs, out[1])
        return out
    _call("mx_grouped_gemm_2d3d_shared_a", "grouped_gemm_2d3d_shared_a", out.device, _ptr(a.codes), _ptr(a.scales),
          _ptr(b.codes), _ptr(b.scales), _ptr(b2.codes), _ptr(b2.scales), _ptr(offs), _ptr(out[0]), _ptr(out[1]),
          T, N, K, G, N, _stream(out))
    return out


def mx_grouped_gemm_2d2d_shared_b(at: MXData, at2: MXData, bt: MXData, offs: torch.Tensor) -> torch.Tensor:
    """bf16 [2, G, N, K]: out[0][g] = at[:, tokens of g] x bt[:, tokens of g]^T and out[1][g] the
    same with at2.  One launch of the persistent kernel when the scales are in MFMA order,
    otherwise two grouped GEMMs; bit-identical either way."""
    N, T = at.codes.shape
    K = bt.codes.shape[0]
    if at2.codes.shape != at.codes.shape or bt.codes.shape[1] != T:
        raise ValueError("operand shapes do not match")
    G = offs.numel()
    out = torch.empty((2, G, N, K), dtype=torch.bfloat16, device=at.codes.device)
    fast = all(d.scale_order == MX_SCALES_MFMA for d in (at, at2, bt))
    if not fast or T == 0 or T % 128 or K % 8:
        mx_grouped_gemm_2d2d(at, bt, offs, out[0])
        mx_grouped_gemm_2d2d(at2, bt, offs, out[1])
        return out
    _call("mx_grouped_gemm_2d2d_shared_b", "grouped_gemm_2d2d_shared_b", out.device, _ptr(at.codes), _ptr(at.scales),
          _ptr(at2.codes), _ptr(at2.scales), _ptr(bt.codes), _ptr(bt.scales), _ptr(offs), _ptr(out[0]), _ptr(out[1]),
          T, N, K, G, _stream(out))
    return out


def mx_grouped_gemm_2d2d(at: MXData, bt: MXData, offs: torch.Tensor,
                         out: torch.Tensor | None = None) -> torch.Tensor:
    """out[g] = deq(at[:, tokens of g]) @ deq(bt[:, tokens of g])^T  ->  [G, N, K] bf16.

    at: codes [N, T], bt: codes [K, T] (column-wise casts), scales of both in the same order.
    Groups may be any multiple of 32 tokens (checked on the device: a violation gives NaN).
    MFMA order: T a multiple of 128 (the token axis may run past the last group) and the
    persistent kernel (csrc/mx_gemm32.hip) runs.
    """
    N, T = at.codes.shape
    K, Tb = bt.codes.shape
    if T != Tb:
        raise ValueError(f"token count mismatch: {T} vs {Tb}")
    if at.scale_order != bt.scale_order:
        raise ValueError("2d2d expects both scale buffers in the same order")
    G = offs.numel()
    if out is None:
        out = torch.empty((G, N, K), dtype=torch.bfloat16, device=at.codes.device)
    else:
        _wrote(out)
    _call("mx_grouped_gemm_2d2d", "grouped_gemm_2d2d", out.device, _ptr(at.codes), _ptr(at.scales), _ptr(bt.codes), _ptr(bt.scales), _ptr(offs), _ptr(out), T, N, K, G, at.scale_order, _stream(out))
    return out


def group_offsets_pad(counts: torch.Tensor, experts_per_rank: int, num_ranks: int, max_len: int,
                      alignment: int):
    """(permuted_indices int64 [max_len], m_sizes int32 [E], m_offsets int32 [E]); one launch."""
    if not counts.is_cuda:
        raise _lib.MXLibraryError("group_offsets_pad runs on the GPU only")
    c32 = counts.to(torch.int32).contiguous()
    perm = torch.empty(max_len, dtype=torch.int64, device=counts.device)
    m_sizes = torch.empty(experts_per_rank, dtype=torch.int32, device=counts.device)
    m_offsets = torch.empty(experts_per_rank, dtype=torch.int32, device=counts.device)
    _call("mx_group_offsets_pad", "group_offsets_pad", counts.device, _ptr(c32), experts_per_rank, num_ranks, max_len, alignment, _ptr(perm), _ptr(m_sizes), _ptr(m_offsets), _stream(counts))
    return perm, m_sizes, m_offsets
