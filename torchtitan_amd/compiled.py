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

What the traced form does not do: share one cast of an activation between sibling linears
(w1 / w3, wq / wk / wv), fuse the SwiGLU gate or the RMSNorm into the casts, or take grouped
(3-D) weights -- those stay eager features.  Shapes need tokens, in_features and out_features
that are multiples of 32.
"""
from __future__ import annotations

import torch

from . import ops
from .ops import MX_SCALES_MFMA, MXData

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
