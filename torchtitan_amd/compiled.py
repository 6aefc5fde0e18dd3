"""The converted linear as opaque custom operators, for blocks wrapped in ``torch.compile``.

The reference compiles every transformer block with ``fullgraph=True``
(torchtitan/models/llama3/parallelize.py:271-284) and expects a converted ``F.linear`` to trace.
The eager path of this package calls the HIP library through ``ctypes`` inside
``autograd.Function``s, which a tracer cannot follow, so while a graph is being traced
``MXFP8TrainingWeight.__torch_function__`` sends ``F.linear`` here instead: one forward and one
backward operator registered with ``torch.library`` (schemas, fake kernels for shape
propagation, an autograd formula), whose bodies run the same casts and GEMMs as the eager
functions.  A compiled block therefore holds the MXFP8 linears as single nodes with no graph
break, and its results equal the eager ones bit for bit when the eager path runs the same
unfused sequence (``fuse_swiglu_cast=False``; the fused block functions are eager-only).

``torch._grouped_mm`` on a converted 3-D weight traces the same way (the reference compiles MoE
blocks too, torchtitan/models/llama4/parallelize.py ``apply_compile``): one forward and one
backward operator that hold the group padding plan, the casts and the grouped GEMMs, with
output shapes that depend on the static sizes only (the padded token axis is the bound
round_up(T + 32 G), never the routed counts), and the index fill of the token-group padding
wrapper is a third operator.

What the traced form does not do: share one cast of an activation between sibling linears
(w1 / w3, wq / wk / wv), fuse the SwiGLU gate or the RMSNorm into the casts, or reuse cached
weight casts -- those stay eager features.  Dense shapes need tokens, in_features and
out_features that are multiples of 32; grouped shapes need K and N multiples of 32.
"""
from __future__ import annotations

import torch

from . import ops
from .mx_tensor import _cast_into_groups, _grouped_2d3d_padded, _pad_plan
from .ops import MX_SCALES_MFMA, MX_SCALES_ROWMAJOR, MXData

_MODE_NAMES = {v: k for k, v in ops.SCALE_MODES.items()}


def _dims(x: torch.Tensor, weight: torch.Tensor):
    K = x.shape[-1]
    M = x.numel() // K if K else 0
    N = weight.shape[0]
    return M, K, N


@torch.library.custom_op("torchtitan_amd::mx_linear_fwd", mutates_args=())
def mx_linear_fwd(x: torch.Tensor, weight: torch.Tensor, mode: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """y = x W^T in MXFP8 plus what the backward needs: the column-wise MXFP8 forms of x
    (codes [K, M], MFMA-order scales) and of W (codes [K, N], MFMA-order scales)."""
    M, K, N = _dims(x, weight)
    name = _MODE_NAMES[mode]
    x2 = x.reshape(M, K)
    if x2.dtype != torch.bfloat16:
        x2 = x2.to(torch.bfloat16)
    w = (weight if weight.dtype == torch.bfloat16 else weight.to(torch.bfloat16)).contiguous()
    xq0, xq1 = ops.to_mx_dim0_dim1(x2.contiguous(), name, MX_SCALES_MFMA)
    wq0, wq1 = ops.to_mx_dim0_dim1(w, name, MX_SCALES_MFMA)
    y = ops.mx_gemm_nt(xq0, wq0).view(*x.shape[:-1], N)
    return y, xq1.codes, xq1.scales, wq1.codes, wq1.scales


@mx_linear_fwd.register_fake
def _(x, weight, mode):
    M, K, N = _dims(x, weight)
    torch._check(K % 32 == 0 and N % 32 == 0, lambda: "the traced MXFP8 linear needs in_features and out_features % 32 == 0")
    torch._check(M % 32 == 0, lambda: "the traced MXFP8 linear needs a multiple of 32 tokens")
    u8 = dict(dtype=torch.uint8, device=x.device)
    return (x.new_empty((*x.shape[:-1], N), dtype=torch.bfloat16),
            torch.empty((K, M), **u8), torch.empty((ops.mfma_scale_bytes(K, M // 32),), **u8),
            torch.empty((K, N), **u8), torch.empty((ops.mfma_scale_bytes(K, N // 32),), **u8))


@torch.library.custom_op("torchtitan_amd::mx_linear_bwd", mutates_args=())
def mx_linear_bwd(dy: torch.Tensor, x_codes_t: torch.Tensor, x_scales_t: torch.Tensor, w_codes_t: torch.Tensor,
                  w_scales_t: torch.Tensor, mode: int, need_dx: bool, need_dw: bool) -> tuple[torch.Tensor, torch.Tensor]:
    """(dX [M, K], dW [N, K]) in bf16 from dY and the saved column-wise forms; an output that is
    not needed comes back empty."""
    K, M = x_codes_t.shape
    N = w_codes_t.shape[1]
    name = _MODE_NAMES[mode]
    dy2 = dy.reshape(M, N)
    if dy2.dtype != torch.bfloat16:
        dy2 = dy2.to(torch.bfloat16)
    dy2 = dy2.contiguous()
    empty = dy2.new_empty((0,))
    if need_dx and need_dw:
        dyq0, dyq1 = ops.to_mx_dim0_dim1(dy2, name, MX_SCALES_MFMA)
    else:
        dyq0 = ops.to_mx_dim0(dy2, name, MX_SCALES_MFMA) if need_dx else None
        dyq1 = ops.to_mx_dim1(dy2, name, MX_SCALES_MFMA) if need_dw else None
    dx = ops.mx_gemm_nt(dyq0, MXData(w_codes_t, w_scales_t, MX_SCALES_MFMA)) if need_dx else empty
    dw = ops.mx_gemm_nt(dyq1, MXData(x_codes_t, x_scales_t, MX_SCALES_MFMA)) if need_dw else empty
    return dx, dw


@mx_linear_bwd.register_fake
def _(dy, x_codes_t, x_scales_t, w_codes_t, w_scales_t, mode, need_dx, need_dw):
    K, M = x_codes_t.shape
    N = w_codes_t.shape[1]
    bf = dict(dtype=torch.bfloat16, device=dy.device)
    return (torch.empty((M, K) if need_dx else (0,), **bf), torch.empty((N, K) if need_dw else (0,), **bf))


def _setup_context(ctx, inputs, output):
    x, weight, mode = inputs
    _, xc, xs, wc, ws = output
    ctx.save_for_backward(xc, xs, wc, ws)
    ctx.mode = mode
    ctx.x_shape, ctx.x_dtype, ctx.w_dtype = x.shape, x.dtype, weight.dtype


def _backward(ctx, gy, *unused):
    xc, xs, wc, ws = ctx.saved_tensors
    need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
    dx, dw = torch.ops.torchtitan_amd.mx_linear_bwd(gy, xc, xs, wc, ws, ctx.mode, need_dx, need_dw)
    gx = dx.view(ctx.x_shape).to(ctx.x_dtype) if need_dx else None
    gw = dw.to(ctx.w_dtype) if need_dw else None
    return gx, gw, None


mx_linear_fwd.register_autograd(_backward, setup_context=_setup_context)


def mx_linear_traced(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, scale_mode: str):
    """``F.linear`` on a converted weight while a graph is being traced.  `weight` and `bias` may
    still be the wrapper subclass: the caller has switched its ``__torch_function__`` off."""
    y = torch.ops.torchtitan_amd.mx_linear_fwd(x, weight, ops.SCALE_MODES[scale_mode])[0]
    if y.dtype != x.dtype:
        y = y.to(x.dtype)
    if bias is not None:
        y = y + bias.to(y.dtype)
    return y


# ----------------------------------------------------------------------------- grouped GEMM
def _grouped_layout(T: int, K: int, N: int, G: int, pad: bool):
    """(scale order, whether the groups are moved to a padded layout, its token count): the
    choices ``_MXGroupedMM.forward`` makes, as a function of the static sizes."""
    fast = K % 128 == 0 and N % 128 == 0 and G <= ops.FAST_MAX_GROUPS
    padded = pad or fast
    step = ops.FAST_LENGTH_MULTIPLE if fast else ops.BLOCK
    Tp = -(-(T + ops.BLOCK * G) // step) * step if padded else T
    return (MX_SCALES_MFMA if fast else MX_SCALES_ROWMAJOR), padded, Tp, (ops.FAST_LENGTH_MULTIPLE if fast else 1)


def _fake_scales(rows: int, nblk: int, order: int, device):
    if order == MX_SCALES_MFMA:
        return torch.empty((ops.mfma_scale_bytes(rows, nblk),), dtype=torch.uint8, device=device)
    return torch.empty((rows, nblk), dtype=torch.uint8, device=device)


@torch.library.custom_op("torchtitan_amd::mx_grouped_mm_fwd", mutates_args=())
def mx_grouped_mm_fwd(x: torch.Tensor, weight: torch.Tensor, offs: torch.Tensor, mode: int, pad: bool) -> tuple[
        torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """y[rows of g] = x[rows of g] W[g]^T for x [T, K], W [G, N, K], offs = inclusive int32 group
    ends; also the plan (padded offsets, gather indices, rows' places in the padded layout; the
    last two empty when the groups stay where they are) and the column-wise MXFP8 forms of the
    padded x (codes [K, Tp]) and of W (codes [G, K, N]) for the backward."""
    T, K = x.shape
    G, N, _ = weight.shape
    name = _MODE_NAMES[mode]
    order, padded, _, multiple = _grouped_layout(T, K, N, G, pad)
    xb = (x if x.dtype == torch.bfloat16 else x.to(torch.bfloat16)).contiguous()
    w = (weight if weight.dtype == torch.bfloat16 else weight.to(torch.bfloat16)).contiguous()
    if padded:
        perm, offs_p, back = _pad_plan(offs, T, ops.BLOCK, multiple)
    else:
        perm = back = None
        offs_p = offs.clone()
    xq0, xq1 = _cast_into_groups(xb, perm, name, order, True)
    wq0, wq1 = ops.to_mx_dim0_dim1_batched(w, name, MX_SCALES_MFMA)
    y = _grouped_2d3d_padded(xq0, wq0, offs_p, back)
    none = torch.empty((0,), dtype=torch.int64, device=x.device)
    return (y, offs_p, perm if padded else none, back if padded else none.clone(),
            xq1.codes, xq1.scales, wq1.codes, wq1.scales)


@mx_grouped_mm_fwd.register_fake
def _(x, weight, offs, mode, pad):
    T, K = x.shape
    G, N, _ = weight.shape
    torch._check(K % 32 == 0 and N % 32 == 0, lambda: "the traced MXFP8 grouped_mm needs K and N % 32 == 0")
    order, padded, Tp, _ = _grouped_layout(T, K, N, G, pad)
    torch._check(Tp % 32 == 0, lambda: "without padding the token dimension must be a multiple of 32")
    dev = x.device
    i64 = dict(dtype=torch.int64, device=dev)
    return (torch.empty((T, N), dtype=torch.bfloat16, device=dev),
            torch.empty((G,), dtype=torch.int32, device=dev),
            torch.empty((Tp if padded else 0,), **i64), torch.empty((T if padded else 0,), **i64),
            torch.empty((K, Tp), dtype=torch.uint8, device=dev), _fake_scales(K, Tp // 32, order, dev),
            torch.empty((G, K, N), dtype=torch.uint8, device=dev),
            torch.empty((G * ops.mfma_scale_bytes(K, N // 32),), dtype=torch.uint8, device=dev))


@torch.library.custom_op("torchtitan_amd::mx_grouped_mm_bwd", mutates_args=())
def mx_grouped_mm_bwd(dy: torch.Tensor, offs_p: torch.Tensor, perm: torch.Tensor, back: torch.Tensor,
                      x_codes_t: torch.Tensor, x_scales_t: torch.Tensor, w_codes_t: torch.Tensor,
                      w_scales_t: torch.Tensor, mode: int, need_dx: bool, need_dw: bool) -> tuple[torch.Tensor, torch.Tensor]:
    """(dX [T, K], dW [G, N, K]) in bf16 from dY [T, N] and what the forward saved; an output
    that is not needed comes back empty."""
    T = dy.shape[0]
    G, K, N = w_codes_t.shape
    name = _MODE_NAMES[mode]
    padded = perm.numel() > 0
    order = MX_SCALES_MFMA if x_scales_t.dim() == 1 else MX_SCALES_ROWMAJOR
    dyb = (dy if dy.dtype == torch.bfloat16 else dy.to(torch.bfloat16)).contiguous()
    empty = dyb.new_empty((0,))
    if padded or (need_dx and need_dw):
        dyq0, dyq1 = _cast_into_groups(dyb, perm if padded else None, name, order, need_dw)
    else:
        dyq0 = ops.to_mx_dim0(dyb, name, order) if need_dx else None
        dyq1 = ops.to_mx_dim1(dyb, name, order) if need_dw else None
    dx = dw = empty
    if need_dx:
        dx = _grouped_2d3d_padded(dyq0, MXData(w_codes_t, w_scales_t, MX_SCALES_MFMA), offs_p, back if padded else None)
    if need_dw:
        dw = ops.mx_grouped_gemm_2d2d(dyq1, MXData(x_codes_t, x_scales_t, order), offs_p)
    return dx, dw


@mx_grouped_mm_bwd.register_fake
def _(dy, offs_p, perm, back, x_codes_t, x_scales_t, w_codes_t, w_scales_t, mode, need_dx, need_dw):
    T = dy.shape[0]
    G, K, N = w_codes_t.shape
    bf = dict(dtype=torch.bfloat16, device=dy.device)
    return (torch.empty((T, K) if need_dx else (0,), **bf), torch.empty((G, N, K) if need_dw else (0,), **bf))


def _grouped_setup_context(ctx, inputs, output):
    x, weight, offs, mode, pad = inputs
    ctx.save_for_backward(*output[1:])
    ctx.mode = mode
    ctx.x_dtype, ctx.w_dtype = x.dtype, weight.dtype


def _grouped_backward(ctx, gy, *unused):
    need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
    dx, dw = torch.ops.torchtitan_amd.mx_grouped_mm_bwd(gy, *ctx.saved_tensors, ctx.mode, need_dx, need_dw)
    return (dx.to(ctx.x_dtype) if need_dx else None, dw.to(ctx.w_dtype) if need_dw else None, None, None, None)


mx_grouped_mm_fwd.register_autograd(_grouped_backward, setup_context=_grouped_setup_context)


def mx_grouped_mm_traced(x: torch.Tensor, w_t: torch.Tensor, offs: torch.Tensor, scale_mode: str, pad: bool):
    """``torch._grouped_mm(x, w_t, offs=offs)`` on a converted weight while a graph is being
    traced; `w_t` [G, K, N] is the transposed view of the parameter and may still be the wrapper
    subclass (the caller has switched its ``__torch_function__`` off)."""
    if x.dim() != 2 or w_t.dim() != 3 or offs is None:
        raise NotImplementedError("MXFP8 grouped_mm supports the 2D x 3D form with offsets only")
    weight = w_t.transpose(-2, -1)
    return torch.ops.torchtitan_amd.mx_grouped_mm_fwd(x, weight, offs.to(torch.int32), ops.SCALE_MODES[scale_mode], pad)[0]


# ----------------------------------------------------------------------------- padding plan
@torch.library.custom_op("torchtitan_amd::group_offsets_pad", mutates_args=())
def group_offsets_pad(counts: torch.Tensor, experts_per_rank: int, num_ranks: int, max_len: int,
                      alignment: int) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """The index fill of the token-group padding wrapper (``ops.group_offsets_pad``) as a graph
    node: (gather indices int64 [max_len], padded sizes int32 [E], padded inclusive offsets)."""
    return ops.group_offsets_pad(counts, experts_per_rank, num_ranks, max_len, alignment)


@group_offsets_pad.register_fake
def _(counts, experts_per_rank, num_ranks, max_len, alignment):
    i32 = dict(dtype=torch.int32, device=counts.device)
    return (torch.empty((max_len,), dtype=torch.int64, device=counts.device),
            torch.empty((experts_per_rank,), **i32), torch.empty((experts_per_rank,), **i32))
