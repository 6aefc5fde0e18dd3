"""Fused blocks on top of the MXFP8 linears: whole SwiGLU feed-forward, expert block and routed
half of an MoE layer as single autograd functions, with the elementwise steps between the GEMMs
(gate, token gather, score multiply, un-sort and combine, and their backward) folded into the
cast kernels.  Each is bit-identical, or identical up to float32 summation order where stated,
to the converted linears around separate bf16 ops
(torchtitan/models/common/feed_forward.py:61-62, models/common/moe/moe.py:59-76,519-555).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F

from . import ops
from .mx_tensor import (MXFP8Config, MXFP8TrainingWeight, _cast_activation, _cast_cache, _cast_cols_padded,
                        _cast_into_groups, _cast_rows_padded, _cast_weight, _grouped_2d3d_padded,
                        _pad_plan, _unwrap)
from .ops import MX_SCALES_MFMA, MX_SCALES_ROWMAJOR, MXData

# ----------------------------------------------------------------------------- SwiGLU + linear
class _MXSwiGLULinear(torch.autograd.Function):
    """y = (silu(h1) * h3) W^T with the gate formed inside the cast kernel: g is never written
    to memory in forward and only its column-wise MXFP8 form is kept for wgrad.  Backward
    returns the gradients the unfused bf16 ops would (silu and the products rounded to bf16
    tensor by tensor, torchtitan/models/common/feed_forward.py:61-62 under autograd)."""

    @staticmethod
    def forward(ctx, h1, h3, weight, cfg: MXFP8Config):
        mode = cfg.scale_mode
        H, N = h1.shape[-1], weight.shape[0]
        a, b = h1.reshape(-1, H), h3.reshape(-1, H)
        w = weight if weight.dtype == torch.bfloat16 else weight.to(torch.bfloat16)
        gq0, gq1, _ = ops.swiglu_to_mx_dim0_dim1(a, b, mode, MX_SCALES_MFMA)
        need_dh = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        wq0, wq1 = _cast_weight(weight, mode, need_dh, cfg)
        y = ops.mx_gemm_nt(gq0, wq0)
        ctx.cfg, ctx.w_dtype, ctx.have_wq1 = cfg, weight.dtype, wq1 is not None
        saved = [h1, h3]
        if ctx.needs_input_grad[2]:
            saved += [gq1.codes, gq1.scales]
        if need_dh:
            saved += [wq1.codes, wq1.scales] if wq1 is not None else [w]
        ctx.save_for_backward(*saved)
        return y.view(*h1.shape[:-1], N)

    @staticmethod
    def backward(ctx, dy):
        mode = ctx.cfg.scale_mode
        need_dh = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        need_dw = ctx.needs_input_grad[2]
        saved = list(ctx.saved_tensors)
        h1, h3 = saved.pop(0), saved.pop(0)
        N = dy.shape[-1]
        dy2 = dy.reshape(-1, N)
        if dy2.dtype != torch.bfloat16:
            dy2 = dy2.to(torch.bfloat16)
        dy2 = dy2.contiguous()
        gq1 = MXData(saved.pop(0), saved.pop(0), MX_SCALES_MFMA) if need_dw else None
        wq1 = None
        if need_dh:
            if ctx.have_wq1:
                wq1 = MXData(saved.pop(0), saved.pop(0), MX_SCALES_MFMA)
            else:
                wq1 = _cast_cols_padded(saved.pop(0), mode)
        if need_dh and need_dw and N % ops.BLOCK == 0:
            dyq0, dyq1 = ops.to_mx_dim0_dim1(dy2, mode, MX_SCALES_MFMA)
        else:
            dyq0 = _cast_rows_padded(dy2, mode) if need_dh else None
            dyq1 = ops.to_mx_dim1(dy2, mode, MX_SCALES_MFMA) if need_dw else None
        dh1 = dh3 = dw = None
        if need_dh:
            dg = ops.mx_gemm_nt(dyq0, wq1).view(h1.shape)
            if ctx.needs_input_grad[1]:
                dh3 = dg * F.silu(h1)
            if ctx.needs_input_grad[0]:
                dh1 = torch.ops.aten.silu_backward(dg * h3, h1)
        if need_dw:
            dw = ops.mx_gemm_nt(dyq1, gq1)
            if dw.dtype != ctx.w_dtype:
                dw = dw.to(ctx.w_dtype)
        return dh1, dh3, dw, None


def swiglu_fusable(h1: torch.Tensor, h3: torch.Tensor, weight: torch.Tensor) -> bool:
    """The fused gate + cast needs bf16 row-contiguous inputs of one shape with 32-aligned token
    and hidden counts (what a converted SwiGLU block produces) and a converted weight."""
    if torch.compiler.is_compiling():  # the fused block functions are eager-only
        return False
    if not isinstance(weight, MXFP8TrainingWeight) or not weight.mx_config.fuse_swiglu_cast:
        return False
    if h1.dtype != torch.bfloat16 or h3.dtype != torch.bfloat16 or h1.shape != h3.shape:
        return False
    H = h1.shape[-1]
    return (h1.is_contiguous() and h3.is_contiguous() and h1.is_cuda and H % ops.BLOCK == 0
            and h1.numel() // max(H, 1) % ops.BLOCK == 0 and h1.numel() > 0)


def mx_swiglu_linear(h1: torch.Tensor, h3: torch.Tensor, weight: torch.Tensor,
                     bias: torch.Tensor | None = None):
    """``F.linear(F.silu(h1) * h3, weight, bias)`` for a converted weight, with the gate computed
    inside the MXFP8 cast.  Callers check `swiglu_fusable` first."""
    y = _MXSwiGLULinear.apply(h1, h3, _unwrap(weight), weight.mx_config)
    if bias is not None:
        y = y + _unwrap(bias).to(y.dtype)
    return y


# ----------------------------------------------------------------------------- whole SwiGLU block
def _bf16(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.bfloat16 else t.to(torch.bfloat16)


def _take(saved, i):
    """MXData (MFMA-order scales) from two neighbouring slots of a saved list."""
    return MXData(saved[i], saved[i + 1], MX_SCALES_MFMA)


# What the SwiGLU block keeps for its backward, by slot (None where a gradient is not needed):
#   0 h1 and h3 stacked [2, M, H]    1, 2 column-wise W2       3, 4 column-wise x     5, 6 column-wise g
#   7, 8 column-wise W1              9, 10 column-wise W3      11 x, 12 rstd, 13 norm weight (norm in front)
FFN_SAVED = 14


def block_pitch_pad(cfg: MXFP8Config, need_dx: bool, need_dw: bool) -> int:
    """Bytes the eager SwiGLU block leaves between the rows of its MXFP8 codes: ops.CODE_PITCH_PAD
    in a training step (every operand is then cast both ways by the kernels that know pitches);
    none with cached weight casts, whose entries other callers read as dense codes."""
    return ops.CODE_PITCH_PAD if need_dx and need_dw and not cfg.cache_weight_casts else 0


def ffn_forward(x2, x_src, w1, w2, w3, cfg: MXFP8Config, need_dx: bool, need_dw: bool, norm_weight=None,
                eps: float = 0.0, pad: int = 0):
    """Forward of the SwiGLU block on a 2-D bf16 activation: (y [M, out], the FFN_SAVED slots).
    `x_src` is the tensor the activation-cast cache is keyed on (None: no sharing of x's cast
    with sibling linears); `pad`: the row pitch padding of every code matrix (the saved ones
    carry it into the backward).  The eager autograd function and the traced operator both run this."""
    mode = cfg.scale_mode
    rstd = None
    if norm_weight is not None:  # RMSNorm in front: normalised inside the cast, rstd kept for its backward
        x2 = x2.contiguous()
        xq0, xq1, rstd, _ = ops.rms_norm_to_mx(x2, _bf16(norm_weight), eps, mode, MX_SCALES_MFMA, pitch_pad=pad)
    elif x_src is not None:
        xq0, xq1 = _cast_activation(x2, x_src, mode, need_cols=need_dw, pitch_pad=pad)
    elif need_dw:
        xq0, xq1 = ops.to_mx_dim0_dim1(x2.contiguous(), mode, MX_SCALES_MFMA, pitch_pad=pad)
    else:
        xq0, xq1 = ops.to_mx_dim0(x2.contiguous(), mode, MX_SCALES_MFMA), None
    w1q0, w1q1 = _cast_weight(w1, mode, need_dx, cfg, pitch_pad=pad)
    w3q0, w3q1 = _cast_weight(w3, mode, need_dx, cfg, pitch_pad=pad)
    w2q0, w2q1 = _cast_weight(w2, mode, need_dx or need_dw, cfg, pitch_pad=pad)
    h13 = ops.mx_gemm_nt_shared_a(xq0, w1q0, w3q0)  # one launch: x's panels fetched once for both
    gq0, gq1, _ = ops.swiglu_to_mx_dim0_dim1(h13[0], h13[1], mode, MX_SCALES_MFMA, pitch_pad=pad)
    y = ops.mx_gemm_nt(gq0, w2q0)
    saved = [None] * FFN_SAVED
    if need_dx or need_dw:
        saved[0:3] = [h13, w2q1.codes, w2q1.scales]
    if need_dw:
        saved[3:7] = [xq1.codes, xq1.scales, gq1.codes, gq1.scales]
    if need_dx:
        saved[7:11] = [w1q1.codes, w1q1.scales, w3q1.codes, w3q1.scales]
        if norm_weight is not None:
            saved[11:14] = [x2, rstd, norm_weight]
    return y, saved


def ffn_backward(dy2, saved, cfg: MXFP8Config, need_x: bool, need_dw1: bool, need_dw2: bool, need_dw3: bool,
                 need_dnw: bool = False, pad: int = 0):
    """(dx [M, in], dW1, dW2, dW3, d norm weight), bf16, None where not asked for; `pad` as the
    forward's."""
    mode = cfg.scale_mode
    h13 = saved[0]
    w2q1 = _take(saved, 1)
    if need_dw2:
        dyq0, dyq1 = ops.to_mx_dim0_dim1(dy2, mode, MX_SCALES_MFMA, pitch_pad=pad)
    else:
        dyq0, dyq1 = ops.to_mx_dim0(dy2, mode, MX_SCALES_MFMA), None
    dg = ops.mx_gemm_nt(dyq0, w2q1)
    (da0, da1), (db0, db1), _ = ops.swiglu_bwd_to_mx_dim0_dim1(dg, h13[0], h13[1], mode, MX_SCALES_MFMA, pitch_pad=pad)
    dx = dw1 = dw2 = dw3 = dnw = None
    if need_dw1 or need_dw2 or need_dw3:
        xq1, gq1 = _take(saved, 3), _take(saved, 5)
        if need_dw1 and need_dw3:
            dw1, dw3 = ops.mx_gemm_nt_shared_b(da1, db1, xq1).unbind(0)  # one launch over x's column-wise form
        elif need_dw1:
            dw1 = ops.mx_gemm_nt(da1, xq1)
        elif need_dw3:
            dw3 = ops.mx_gemm_nt(db1, xq1)
        if need_dw2:
            dw2 = ops.mx_gemm_nt(dyq1, gq1)
    if need_x or need_dnw:
        # dx = d(h1) W1 + d(h3) W3 as one GEMM: summed in float32, rounded once
        dx = ops.mx_gemm_nt_pair(da0, _take(saved, 7), db0, _take(saved, 9))
        if saved[11] is not None:
            dx, dnw = _rms_norm_backward(dx, saved[11], saved[12], saved[13], need_x, need_dnw)
    return dx, dw1, dw2, dw3, dnw


class _MXFeedForward(torch.autograd.Function):
    """y = (silu(x W1^T) * (x W3^T)) W2^T with every elementwise step folded into a cast kernel.

    Forward: one cast of x, the gate inside the cast that feeds W2.  Backward: the gate's
    gradients inside the cast that feeds the dgrad / wgrad GEMMs of W1 and W3.  Neither g nor
    dh1 / dh3 is written to memory; kept for backward are h1, h3 and the column-wise MXFP8 forms
    of x, g and the weights.  Results are bit-identical to the three converted linears around
    bf16 ``F.silu`` and ``*`` (torchtitan/models/common/feed_forward.py:61-62)."""

    @staticmethod
    def forward(ctx, x, w1, w2, w3, cfg: MXFP8Config, norm_weight=None, eps: float = 0.0):
        need_dx = ctx.needs_input_grad[0] or ctx.needs_input_grad[5]
        need_dw = any(ctx.needs_input_grad[1:4])
        ctx.pad = block_pitch_pad(cfg, need_dx, need_dw)
        y, saved = ffn_forward(x.reshape(-1, x.shape[-1]), x, w1, w2, w3, cfg, need_dx, need_dw, norm_weight, eps,
                               pad=ctx.pad)
        ctx.cfg, ctx.x_shape = cfg, x.shape
        ctx.w_dtypes = (w1.dtype, w2.dtype, w3.dtype)
        ctx.save_for_backward(*saved)
        return y.view(*x.shape[:-1], w2.shape[0])

    @staticmethod
    def backward(ctx, dy):
        _cast_cache.clear()  # the forward that shared x's cast with a sibling is over
        need = ctx.needs_input_grad
        dy2 = _bf16(dy.reshape(-1, dy.shape[-1])).contiguous()
        dx, dw1, dw2, dw3, dnw = ffn_backward(dy2, list(ctx.saved_tensors), ctx.cfg, need[0], need[1], need[2],
                                              need[3], need[5], pad=ctx.pad)
        cast_back = lambda g, dt: g if g is None or g.dtype == dt else g.to(dt)
        if dx is not None:
            dx = dx.view(ctx.x_shape)
        return (dx, cast_back(dw1, ctx.w_dtypes[0]), cast_back(dw2, ctx.w_dtypes[1]), cast_back(dw3, ctx.w_dtypes[2]),
                None, dnw, None)


def feed_forward_fusable(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor) -> bool:
    """The whole-block function needs all three weights converted with gate fusion on, a bf16
    GPU activation and 32-aligned token, model and hidden sizes."""
    ws = (w1, w2, w3)
    if not all(isinstance(w, MXFP8TrainingWeight) and w.mx_config.fuse_swiglu_cast for w in ws):
        return False
    if w1.mx_config.scale_mode != w2.mx_config.scale_mode or w1.mx_config.scale_mode != w3.mx_config.scale_mode:
        return False
    if x.dtype != torch.bfloat16 or not x.is_cuda or x.numel() == 0 or w1.shape != w3.shape:
        return False
    D, H = x.shape[-1], w1.shape[0]
    return D % ops.BLOCK == 0 and H % ops.BLOCK == 0 and (x.numel() // D) % ops.BLOCK == 0


def mx_feed_forward(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor,
                    bias2: torch.Tensor | None = None):
    """``F.linear(F.silu(F.linear(x, w1)) * F.linear(x, w3), w2, bias2)`` for converted weights.
    Callers check `feed_forward_fusable` first."""
    if torch.compiler.is_compiling():  # the same function as one node of the graph (compiled.py)
        from .compiled import mx_feed_forward_traced

        with torch._C.DisableTorchFunctionSubclass():
            return mx_feed_forward_traced(x, w1, w2, w3, bias2)
    y = _MXFeedForward.apply(x, _unwrap(w1), _unwrap(w2), _unwrap(w3), w2.mx_config, None, 0.0)
    if bias2 is not None:
        y = y + _unwrap(bias2).to(y.dtype)
    return y


# ----------------------------------------------------------------------------- RMSNorm in front
def _rms_norm_backward(dh, x2, rstd, norm_weight, need_dx: bool, need_dw: bool):
    """(dx, dweight) of y = rms_norm(x) * weight from dy = dh, with torch's own fused backward
    kernel fed the rstd the forward kernel produced."""
    gx, gw = torch.ops.aten._fused_rms_norm_backward(dh, x2, [x2.shape[-1]], rstd.view(-1, 1), norm_weight,
                                                     [need_dx, need_dw])
    return (gx if need_dx else None), (gw if need_dw else None)


class _MXNormLinears(torch.autograd.Function):
    """(rms_norm(x) W_0^T, rms_norm(x) W_1^T, ...) for linears that share one normalised input
    (wq / wk / wv behind the attention norm): the norm runs inside the one cast that feeds all of
    them; the normalised activation is never written.  Not bit-identical to a separate norm: the
    float32 row reduction differs from torch's in its last bits (a few bf16 values in a million
    move by one step)."""

    @staticmethod
    def forward(ctx, x, norm_weight, eps, cfg: MXFP8Config, *weights):
        mode = cfg.scale_mode
        D = x.shape[-1]
        x2 = x.reshape(-1, D).contiguous()
        hq0, hq1, rstd, _ = ops.rms_norm_to_mx(x2, _bf16(norm_weight), eps, mode, MX_SCALES_MFMA)
        need_dh = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        outs, saved = [], [x2, rstd, norm_weight, hq1.codes, hq1.scales]
        for w in weights:
            wq0, wq1 = _cast_weight(w, mode, need_dh, cfg)
            outs.append(ops.mx_gemm_nt(hq0, wq0).view(*x.shape[:-1], w.shape[0]))
            if need_dh:
                saved += [wq1.codes, wq1.scales]
        ctx.cfg, ctx.x_shape, ctx.need_dh = cfg, x.shape, need_dh
        ctx.w_dtypes = tuple(w.dtype for w in weights)
        ctx.save_for_backward(*saved)
        return tuple(outs)

    @staticmethod
    def backward(ctx, *dys):
        mode = ctx.cfg.scale_mode
        saved = list(ctx.saved_tensors)
        x2, rstd, norm_weight = saved[:3]
        hq1 = MXData(saved[3], saved[4], MX_SCALES_MFMA)
        rest = saved[5:]
        dh, dws = None, []
        for i, dy in enumerate(dys):
            need_dw = ctx.needs_input_grad[4 + i]
            if dy is None or not (ctx.need_dh or need_dw):
                dws.append(None)
                continue
            dy2 = _bf16(dy.reshape(-1, dy.shape[-1])).contiguous()
            if ctx.need_dh and need_dw:
                dyq0, dyq1 = ops.to_mx_dim0_dim1(dy2, mode, MX_SCALES_MFMA)
            else:
                dyq0 = ops.to_mx_dim0(dy2, mode, MX_SCALES_MFMA) if ctx.need_dh else None
                dyq1 = ops.to_mx_dim1(dy2, mode, MX_SCALES_MFMA) if need_dw else None
            if ctx.need_dh:
                part = ops.mx_gemm_nt(dyq0, MXData(rest[2 * i], rest[2 * i + 1], MX_SCALES_MFMA))
                dh = part if dh is None else dh + part
            dw = None
            if need_dw:
                dw = ops.mx_gemm_nt(dyq1, hq1)
                if dw.dtype != ctx.w_dtypes[i]:
                    dw = dw.to(ctx.w_dtypes[i])
            dws.append(dw)
        dx = dnw = None
        if ctx.need_dh and dh is not None:
            dx, dnw = _rms_norm_backward(dh, x2, rstd, norm_weight, ctx.needs_input_grad[0], ctx.needs_input_grad[1])
            if dx is not None:
                dx = dx.view(ctx.x_shape)
        return (dx, dnw, None, None, *dws)


def norm_fusable(x: torch.Tensor, norm_weight: torch.Tensor | None, *weights: torch.Tensor,
                 for_feed_forward: bool = False) -> bool:
    """RMSNorm can move into the cast when the converter was built with `fuse_rmsnorm_cast`, the
    norm has a bf16 weight, every linear behind it is converted with in_features % 32 == 0 and
    out_features % 32 == 0, and x is a bf16 GPU tensor with a multiple of 32 tokens.
    `for_feed_forward`: the caller is about to use `mx_norm_feed_forward`, which also exists as a
    traced operator; `mx_norm_linears` is an eager function only."""
    if torch.compiler.is_compiling() and not for_feed_forward:
        return False  # of the two norm fusions only the feed-forward block has a traced operator
    if norm_weight is None or norm_weight.dtype != torch.bfloat16 or not weights:
        return False
    if not all(isinstance(w, MXFP8TrainingWeight) and w.mx_config.fuse_rmsnorm_cast and w.dim() == 2 for w in weights):
        return False
    if x.dtype != torch.bfloat16 or not x.is_cuda or x.numel() == 0:
        return False
    D = x.shape[-1]
    if any(w.shape[1] != D or w.shape[0] % ops.BLOCK for w in weights):
        return False
    return D % ops.BLOCK == 0 and (x.numel() // D) % ops.BLOCK == 0 and norm_weight.shape == (D,)


def _norm_eps(x: torch.Tensor, eps: float | None) -> float:
    # nn.RMSNorm(eps=None) means the machine epsilon of the input's dtype
    return float(torch.finfo(x.dtype).eps if eps is None else eps)


def mx_norm_linears(x: torch.Tensor, norm_weight: torch.Tensor, eps: float | None, weights) -> tuple:
    """``tuple(F.linear(F.rms_norm(x, (dim,), norm_weight, eps), w) for w in weights)`` for
    converted weights without biases.  Callers check `norm_fusable` first."""
    weights = list(weights)
    return _MXNormLinears.apply(x, norm_weight, _norm_eps(x, eps), weights[0].mx_config,
                                *[_unwrap(w) for w in weights])


def mx_norm_feed_forward(x: torch.Tensor, norm_weight: torch.Tensor, eps: float | None, w1: torch.Tensor,
                         w2: torch.Tensor, w3: torch.Tensor, bias2: torch.Tensor | None = None):
    """The SwiGLU block applied to ``F.rms_norm(x, (dim,), norm_weight, eps)``, norm inside the
    cast.  Callers check `norm_fusable(x, norm_weight, w1, w3)` and `feed_forward_fusable`."""
    if torch.compiler.is_compiling():
        from .compiled import mx_feed_forward_traced

        with torch._C.DisableTorchFunctionSubclass():
            return mx_feed_forward_traced(x, w1, w2, w3, bias2, norm_weight, _norm_eps(x, eps))
    y = _MXFeedForward.apply(x, _unwrap(w1), _unwrap(w2), _unwrap(w3), w2.mx_config, norm_weight,
                             _norm_eps(x, eps))
    if bias2 is not None:
        y = y + _unwrap(bias2).to(y.dtype)
    return y


def grouped_layout(D: int, H: int, G: int):
    """(scale order of the activations, multiple the padded token axis is rounded up to) for an
    expert block of model size D and hidden size H: the persistent kernel with MFMA-order scales
    where it takes the shape, the general grouped kernels with row-major scales otherwise."""
    fast = D % 128 == 0 and H % 128 == 0 and G <= ops.FAST_MAX_GROUPS
    return (MX_SCALES_MFMA if fast else MX_SCALES_ROWMAJOR), (ops.FAST_LENGTH_MULTIPLE if fast else 1), fast


# What the expert block keeps for its backward, by slot (None where not needed):
#   0 padded group ends   1 gather indices, 2 the way back (`_pad_plan`: rows' places in the padded
#   layout, int64 [T], or the unpadded group ends, int32 [G], when the GEMMs write unpadded rows)
#   3 h1 and h3 stacked [2, Tp, H]   4, 5 column-wise W2   6, 7 column-wise x   8, 9 column-wise g
#   10, 11 column-wise W1            12, 13 column-wise W3
GROUPED_FFN_SAVED = 14


def grouped_ffn_forward(x, w1, w2, w3, offs, cfg: MXFP8Config, need_dx: bool, need_dw: bool):
    """Forward of the expert block on x [T, D] (bf16): (y [T, D], the GROUPED_FFN_SAVED slots)."""
    mode = cfg.scale_mode
    T, D = x.shape
    G, H, _ = w1.shape
    order, multiple, fast = grouped_layout(D, H, G)
    perm = back = None
    if cfg.pad_token_groups_for_grouped_mm or fast:
        perm, offs_p, back = _pad_plan(offs, T, ops.BLOCK, multiple, direct=fast)
    else:
        offs_p = offs
        if T % ops.BLOCK:
            raise ValueError("without padding the token dimension must be a multiple of 32")
    xq0, xq1 = _cast_into_groups(x.contiguous(), perm, mode, order, need_dw)
    w1q0, w1q1 = _cast_weight(w1, mode, need_dx, cfg)
    w3q0, w3q1 = _cast_weight(w3, mode, need_dx, cfg)
    w2q0, w2q1 = _cast_weight(w2, mode, need_dx or need_dw, cfg)
    h13 = ops.mx_grouped_gemm_2d3d_shared_a(xq0, w1q0, w3q0, offs_p)  # one pass over the routed tokens
    gq0, gq1, _ = ops.swiglu_to_mx_dim0_dim1(h13[0], h13[1], mode, order)
    y = _grouped_2d3d_padded(gq0, w2q0, offs_p, back, T)
    saved = [None] * GROUPED_FFN_SAVED
    saved[0:3] = [offs_p, perm, back]
    if need_dx or need_dw:
        saved[3:6] = [h13, w2q1.codes, w2q1.scales]
    if need_dw:
        saved[6:10] = [xq1.codes, xq1.scales, gq1.codes, gq1.scales]
    if need_dx:
        saved[10:14] = [w1q1.codes, w1q1.scales, w3q1.codes, w3q1.scales]
    return y, saved


def grouped_ffn_backward(dy, saved, cfg: MXFP8Config, order: int, need_dx: bool, need_dw1: bool, need_dw2: bool,
                         need_dw3: bool):
    """(dx [T, D], dW1, dW2, dW3), bf16, None where not asked for; dy [T, D] bf16 contiguous."""
    mode = cfg.scale_mode
    offs_p, perm, back, h13 = saved[0:4]
    w2q1 = _take(saved, 4)
    dyq0, dyq1 = _cast_into_groups(dy, perm, mode, order, need_dw2)
    dg = ops.mx_grouped_gemm_2d3d(dyq0, w2q1, offs_p)
    (da0, da1), (db0, db1), _ = ops.swiglu_bwd_to_mx_dim0_dim1(dg, h13[0], h13[1], mode, order)
    dx = dw1 = dw2 = dw3 = None
    if need_dw1 or need_dw2 or need_dw3:
        xq1, gq1 = MXData(saved[6], saved[7], order), MXData(saved[8], saved[9], order)
        if need_dw1 and need_dw3:
            dw1, dw3 = ops.mx_grouped_gemm_2d2d_shared_b(da1, db1, xq1, offs_p).unbind(0)
        elif need_dw1:
            dw1 = ops.mx_grouped_gemm_2d2d(da1, xq1, offs_p)
        elif need_dw3:
            dw3 = ops.mx_grouped_gemm_2d2d(db1, xq1, offs_p)
        if need_dw2:
            dw2 = ops.mx_grouped_gemm_2d2d(dyq1, gq1, offs_p)
    if need_dx:
        w1q1, w3q1 = _take(saved, 10), _take(saved, 12)
        # d(h1) W1[g] + d(h3) W3[g] as one grouped GEMM (summed in float32, rounded once)
        dx = _grouped_2d3d_padded(da0, w1q1, offs_p, back, dy.shape[0], db0, w3q1)
    return dx, dw1, dw2, dw3


class _MXGroupedFeedForward(torch.autograd.Function):
    """The expert block ``grouped_mm(silu(grouped_mm(x, w1)) * grouped_mm(x, w3), w2)`` as one
    function (torchtitan/models/common/moe/moe.py:59-76): tokens are moved into aligned groups
    once instead of once per GEMM, x is cast once for w1 and w3, and the gate and its backward
    run inside the cast kernels as in `_MXFeedForward`.  Bit-identical to the three converted
    grouped GEMMs around bf16 ``F.silu`` and ``*``."""

    @staticmethod
    def forward(ctx, x, w1, w2, w3, offs, cfg: MXFP8Config):
        need_dx = ctx.needs_input_grad[0]
        need_dw = any(ctx.needs_input_grad[1:4])
        y, saved = grouped_ffn_forward(_bf16(x), w1, w2, w3, offs, cfg, need_dx, need_dw)
        ctx.cfg = cfg
        ctx.order = grouped_layout(x.shape[1], w1.shape[1], w1.shape[0])[0]
        ctx.dtypes = (x.dtype, w1.dtype, w2.dtype, w3.dtype)
        ctx.save_for_backward(*saved)
        return y

    @staticmethod
    def backward(ctx, dy):
        need = ctx.needs_input_grad
        grads = grouped_ffn_backward(_bf16(dy).contiguous(), list(ctx.saved_tensors), ctx.cfg, ctx.order, need[0],
                                     need[1], need[2], need[3])
        dx, dw1, dw2, dw3 = (g if g is None or g.dtype == dt else g.to(dt) for g, dt in zip(grads, ctx.dtypes))
        return dx, dw1, dw2, dw3, None, None


def grouped_experts_align_themselves(w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor) -> bool:
    """All three expert parameters converted with token-group padding on: their grouped GEMMs
    take groups of any size, so nothing has to pad the groups around them."""
    return all(isinstance(w, MXFP8TrainingWeight) and w.dim() == 3
               and w.mx_config.pad_token_groups_for_grouped_mm for w in (w1, w2, w3))


def grouped_feed_forward_fusable(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                                 w3: torch.Tensor) -> bool:
    """All three expert parameters converted with gate fusion on, a 2-D GPU activation, model
    and hidden sizes multiples of 32."""
    ws = (w1, w2, w3)
    if not all(isinstance(w, MXFP8TrainingWeight) and w.mx_config.fuse_swiglu_cast and w.dim() == 3 for w in ws):
        return False
    if x.dim() != 2 or not x.is_cuda or x.numel() == 0 or w1.shape != w3.shape:
        return False
    if w1.mx_config.scale_mode != w2.mx_config.scale_mode or w1.mx_config.scale_mode != w3.mx_config.scale_mode:
        return False
    return x.shape[-1] % ops.BLOCK == 0 and w1.shape[1] % ops.BLOCK == 0


def mx_grouped_feed_forward(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor,
                            offs: torch.Tensor):
    """The SwiGLU expert block for converted 3-D parameters w1, w3 [G, hidden, dim] and
    w2 [G, dim, hidden]; offs = inclusive cumulative group sizes.  Returns bf16.
    Callers check `grouped_feed_forward_fusable` first."""
    if torch.compiler.is_compiling():
        from .compiled import mx_grouped_feed_forward_traced

        with torch._C.DisableTorchFunctionSubclass():
            return mx_grouped_feed_forward_traced(x, w1, w2, w3, offs)
    return _MXGroupedFeedForward.apply(x, _unwrap(w1), _unwrap(w2), _unwrap(w3), offs.to(torch.int32),
                                       w2.mx_config)


# What the routed half of an MoE layer keeps for its backward, by slot (None where not needed):
#   0 padded group ends   1 token of every padded row   2 score of every padded row   3 padded row of every
#   (token, choice) pair [T, k]   4 scores (float32)   5 h1 and h3 stacked   6, 7 column-wise W2
#   8, 9 column-wise x    10, 11 column-wise g    12, 13 column-wise W1    14, 15 column-wise W3
#   16 x (scores in front of the experts) or the padded expert outputs (scores behind them)
ROUTED_SAVED = 17


def routed_forward(x, top_scores, w1, w2, w3, tok_sorted, counts, score_before: bool, cfg: MXFP8Config,
                   need_dx: bool, need_ds: bool, need_dw: bool):
    """Forward of the routed half on x [T, D] (bf16 contiguous): (out [T, D], the ROUTED_SAVED slots)."""
    mode = cfg.scale_mode
    T, D = x.shape
    k = top_scores.shape[1]
    G, H, _ = w1.shape
    scores = top_scores.float().contiguous()
    order, multiple, _ = grouped_layout(D, H, G)
    # aligned group layout and the maps between padded rows, tokens and (token, j) pairs
    offs_p, src_row, row_score, pos = ops.moe_route_plan(counts, tok_sorted, scores.view(-1), k, ops.BLOCK, multiple)
    pos = pos.view(T, k)
    xq0, xq1 = ops.to_mx_rows_gathered(x, src_row, mode, order, need_dw, row_score if score_before else None)
    need_dg = need_dx or need_ds or need_dw
    w1q0, w1q1 = _cast_weight(w1, mode, need_dx or need_ds, cfg)
    w3q0, w3q1 = _cast_weight(w3, mode, need_dx or need_ds, cfg)
    w2q0, w2q1 = _cast_weight(w2, mode, need_dg, cfg)
    h13 = ops.mx_grouped_gemm_2d3d_shared_a(xq0, w1q0, w3q0, offs_p)  # one pass over the routed tokens
    gq0, gq1, _ = ops.swiglu_to_mx_dim0_dim1(h13[0], h13[1], mode, order)
    yp = ops.mx_grouped_gemm_2d3d(gq0, w2q0, offs_p)
    out = ops.moe_combine(yp, pos, None if score_before else scores)
    saved = [None] * ROUTED_SAVED
    saved[0:5] = [offs_p, src_row, row_score, pos, scores]
    if need_dg:
        saved[5:8] = [h13, w2q1.codes, w2q1.scales]
    if need_dw:
        saved[8:12] = [xq1.codes, xq1.scales, gq1.codes, gq1.scales]
    if need_dx or need_ds:
        saved[12:16] = [w1q1.codes, w1q1.scales, w3q1.codes, w3q1.scales]
    if need_ds:
        saved[16] = x if score_before else yp
    return out, saved


def routed_backward(dout, saved, cfg: MXFP8Config, order: int, score_before: bool, need_dx: bool, need_ds: bool,
                    need_dw1: bool, need_dw2: bool, need_dw3: bool):
    """(dx [T, D] bf16, d scores [T, k] float32, dW1, dW2, dW3 bf16), None where not asked for."""
    mode = cfg.scale_mode
    offs_p, src_row, row_score, pos, scores, h13 = saved[0:6]
    T, k = pos.shape
    w2q1 = _take(saved, 6)
    # gradient of the padded expert outputs: dout of the row's token (times its score)
    dyq0, dyq1 = ops.to_mx_rows_gathered(dout, src_row, mode, order, need_dw2, None if score_before else row_score)
    dg = ops.mx_grouped_gemm_2d3d(dyq0, w2q1, offs_p)
    (da0, da1), (db0, db1), _ = ops.swiglu_bwd_to_mx_dim0_dim1(dg, h13[0], h13[1], mode, order)
    dx = ds = dw1 = dw2 = dw3 = None
    if need_dw1 or need_dw2 or need_dw3:
        xq1, gq1 = MXData(saved[8], saved[9], order), MXData(saved[10], saved[11], order)
        if need_dw1 and need_dw3:
            dw1, dw3 = ops.mx_grouped_gemm_2d2d_shared_b(da1, db1, xq1, offs_p).unbind(0)
        elif need_dw1:
            dw1 = ops.mx_grouped_gemm_2d2d(da1, xq1, offs_p)
        elif need_dw3:
            dw3 = ops.mx_grouped_gemm_2d2d(db1, xq1, offs_p)
        if need_dw2:
            dw2 = ops.mx_grouped_gemm_2d2d(dyq1, gq1, offs_p)
    if need_dx or need_ds:
        w1q1, w3q1 = _take(saved, 12), _take(saved, 14)
        if need_dx or (need_ds and score_before):
            # gradient of the (scaled) routed inputs, padded layout: the halves from w1 and
            # w3 summed inside one grouped GEMM (float32, one rounding)
            dxp = ops.mx_grouped_gemm_2d3d_pair(da0, w1q1, db0, w3q1, offs_p)
        if need_dx:
            dx = ops.moe_combine(dxp, pos, scores if score_before else None)
        if need_ds:
            other = saved[16]  # x (scores in front of the experts) or the expert outputs
            token = torch.arange(T * k, device=pos.device, dtype=torch.int64).div_(k, rounding_mode="floor")
            if score_before:
                ds = ops.moe_row_dot(dxp, pos.view(-1), other, token)
            else:
                ds = ops.moe_row_dot(other, pos.view(-1), dout, token)
            ds = ds.view(T, k)
    return dx, ds, dw1, dw2, dw3


class _MXRoutedExperts(torch.autograd.Function):
    """The routed half of an MoE layer as one function (torchtitan/models/common/moe/moe.py:519-555):

        out[t] = sum_j  c[t, j] * experts(x[t] * r[t, j])        j over the token's top_k experts

    with r = scores, c = 1 when the scores multiply the expert inputs (`score_before_experts`)
    and r = 1, c = scores otherwise.  The token gather, the score multiply and the move into
    aligned expert groups happen inside the cast kernel (no routed copy of x exists); the
    un-sort and the weighted sum over top_k are one kernel over the padded expert outputs; in
    backward the same two kernels swap roles and the score gradients are row dot products."""

    @staticmethod
    def forward(ctx, x, top_scores, w1, w2, w3, tok_sorted, counts, score_before: bool, cfg: MXFP8Config):
        need_dx, need_ds = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_dw = any(ctx.needs_input_grad[2:5])
        out, saved = routed_forward(_bf16(x).contiguous(), top_scores, w1, w2, w3, tok_sorted, counts, score_before,
                                    cfg, need_dx, need_ds, need_dw)
        ctx.cfg, ctx.score_before = cfg, score_before
        ctx.order = grouped_layout(x.shape[1], w1.shape[1], w1.shape[0])[0]
        ctx.dtypes = (x.dtype, top_scores.dtype, w1.dtype, w2.dtype, w3.dtype)
        ctx.save_for_backward(*saved)
        return out

    @staticmethod
    def backward(ctx, dout):
        need = ctx.needs_input_grad
        grads = routed_backward(_bf16(dout).contiguous(), list(ctx.saved_tensors), ctx.cfg, ctx.order,
                                ctx.score_before, need[0], need[1], need[2], need[3], need[4])
        dx, ds, dw1, dw2, dw3 = (g if g is None or g.dtype == dt else g.to(dt) for g, dt in zip(grads, ctx.dtypes))
        return dx, ds, dw1, dw2, dw3, None, None, None, None


def mx_routed_experts(x: torch.Tensor, top_scores: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor,
                      w3: torch.Tensor, token_indices_experts_sorted: torch.Tensor,
                      num_tokens_per_expert: torch.Tensor, score_before_experts: bool) -> torch.Tensor:
    """Gather, score, run the SwiGLU experts and combine, for converted expert parameters.
    x [T, dim] bf16, top_scores [T, top_k]; the index tensor is the stable argsort of the
    flattened expert choices.  Callers check `grouped_feed_forward_fusable` first."""
    if torch.compiler.is_compiling():
        from .compiled import mx_routed_experts_traced

        with torch._C.DisableTorchFunctionSubclass():
            return mx_routed_experts_traced(x, top_scores, w1, w2, w3, token_indices_experts_sorted,
                                            num_tokens_per_expert, score_before_experts)
    return _MXRoutedExperts.apply(x, top_scores, _unwrap(w1), _unwrap(w2), _unwrap(w3),
                                  token_indices_experts_sorted, num_tokens_per_expert,
                                  bool(score_before_experts), w2.mx_config)
