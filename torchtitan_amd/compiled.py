"""The converted linear as opaque custom operators, for blocks wrapped in ``torch.compile``.

The reference compiles every transformer block with ``fullgraph=True``
(torchtitan/models/llama3/parallelize.py:271-284) and expects a converted ``F.linear`` to trace.
The eager path of this package calls the HIP library through ``ctypes`` inside
``autograd.Function``s, which a tracer cannot follow, so while a graph is being traced
``MXFP8TrainingWeight.__torch_function__`` sends ``F.linear`` here instead: one forward and one
backward operator registered with ``torch.library`` (schemas, fake kernels for shape
propagation, an autograd formula), whose bodies run the same casts and GEMMs as the eager
functions.  A compiled block therefore holds the MXFP8 linears as single nodes with no graph
break, and its results equal the eager ones bit for bit.

``torch._grouped_mm`` on a converted 3-D weight traces the same way (the reference compiles MoE
blocks too, torchtitan/models/llama4/parallelize.py ``apply_compile``): one forward and one
backward operator that hold the group padding plan, the casts and the grouped GEMMs, with
output shapes that depend on the static sizes only (the padded token axis is the bound
round_up(T + 32 G), never the routed counts), and the index fill of the token-group padding
wrapper is a third operator.

The fused block functions (SwiGLU feed-forward block with the gate inside the casts, optionally
with the RMSNorm in front of it; the expert block; the routed half of an MoE layer) are operators
of the same kind further down: a compiled block runs the kernel sequence the eager path runs.
What the traced form does not do: share one cast of an activation between sibling linears
outside those blocks (wq / wk / wv), or fuse the RMSNorm in front of them (`mx_norm_linears`).
Without gradients (``torch.no_grad()``, inputs that need none) the column-wise casts are left
out; weights converted with ``cache_weight_casts`` take their casts from the cache.  Dense
shapes need tokens, in_features and out_features that are multiples of 32; grouped shapes need
K and N multiples of 32.
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
def mx_linear_fwd(x: torch.Tensor, weight: torch.Tensor, mode: int, need_dx: bool = True, need_dw: bool = True,
                  cache_w: bool = False) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """y = x W^T in MXFP8 plus what the backward needs: the column-wise MXFP8 forms of x
    (codes [K, M], MFMA-order scales; empty unless `need_dw`) and of W (codes [K, N], MFMA-order
    scales; empty unless `need_dx`).  Without gradients only the row-wise casts run.  `cache_w`:
    the weight's casts come from, and go to, the cache of unchanged weights."""
    from .mx_tensor import _cast_weight

    M, K, N = _dims(x, weight)
    name = _MODE_NAMES[mode]
    x2 = x.reshape(M, K)
    if x2.dtype != torch.bfloat16:
        x2 = x2.to(torch.bfloat16)
    x2 = x2.contiguous()
    if need_dw:
        xq0, xq1 = ops.to_mx_dim0_dim1(x2, name, MX_SCALES_MFMA)
    else:
        xq0, xq1 = ops.to_mx_dim0(x2, name, MX_SCALES_MFMA), None
    wq0, wq1 = _cast_weight(weight, name, need_dx, _block_cfg(mode, cache_w))
    y = ops.mx_gemm_nt(xq0, wq0).view(*x.shape[:-1], N)
    if cache_w and wq1 is not None:  # an operator's outputs are its own: not the cache's tensors
        wq1 = MXData(wq1.codes.clone(), wq1.scales.clone(), MX_SCALES_MFMA)
    e = lambda: _empty(x.device)
    return (y, xq1.codes if need_dw else e(), xq1.scales if need_dw else e(),
            wq1.codes if need_dx else e(), wq1.scales if need_dx else e())


@mx_linear_fwd.register_fake
def _(x, weight, mode, need_dx=True, need_dw=True, cache_w=False):
    M, K, N = _dims(x, weight)
    torch._check(K % 32 == 0 and N % 32 == 0, lambda: "the traced MXFP8 linear needs in_features and out_features % 32 == 0")
    torch._check(M % 32 == 0, lambda: "the traced MXFP8 linear needs a multiple of 32 tokens")
    dev = x.device
    return (x.new_empty((*x.shape[:-1], N), dtype=torch.bfloat16),
            _u8((K, M), dev) if need_dw else _empty(dev), _mfma(K, M // 32, dev) if need_dw else _empty(dev),
            _u8((K, N), dev) if need_dx else _empty(dev), _mfma(K, N // 32, dev) if need_dx else _empty(dev))


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
    x, weight, mode = inputs[:3]
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
    return gx, gw, None, None, None, None


mx_linear_fwd.register_autograd(_backward, setup_context=_setup_context)


def mx_linear_traced(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, scale_mode: str,
                     cache_w: bool = False):
    """``F.linear`` on a converted weight while a graph is being traced.  `weight` and `bias` may
    still be the wrapper subclass: the caller has switched its ``__torch_function__`` off."""
    grads = torch.is_grad_enabled()
    y = torch.ops.torchtitan_amd.mx_linear_fwd(x, weight, ops.SCALE_MODES[scale_mode], grads and x.requires_grad,
                                               grads and weight.requires_grad, cache_w)[0]
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
    ends; also the plan (padded offsets, gather indices, the way back -- rows' places in the
    padded layout, or the unpadded group ends as int32 where the GEMM writes unpadded rows; the
    last two empty when the groups stay where they are) and the column-wise MXFP8 forms of the
    padded x (codes [K, Tp]) and of W (codes [G, K, N]) for the backward."""
    T, K = x.shape
    G, N, _ = weight.shape
    name = _MODE_NAMES[mode]
    order, padded, _, multiple = _grouped_layout(T, K, N, G, pad)
    xb = (x if x.dtype == torch.bfloat16 else x.to(torch.bfloat16)).contiguous()
    w = (weight if weight.dtype == torch.bfloat16 else weight.to(torch.bfloat16)).contiguous()
    if padded:
        perm, offs_p, back = _pad_plan(offs, T, ops.BLOCK, multiple, direct=order == MX_SCALES_MFMA)
    else:
        perm = back = None
        offs_p = offs.clone()
    xq0, xq1 = _cast_into_groups(xb, perm, name, order, True)
    wq0, wq1 = ops.to_mx_dim0_dim1_batched(w, name, MX_SCALES_MFMA)
    y = _grouped_2d3d_padded(xq0, wq0, offs_p, back, T)
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
            torch.empty((Tp if padded else 0,), **i64),
            (torch.empty((G,), dtype=torch.int32, device=dev) if padded and order == MX_SCALES_MFMA
             else torch.empty((T if padded else 0,), **i64)),
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
        dx = _grouped_2d3d_padded(dyq0, MXData(w_codes_t, w_scales_t, MX_SCALES_MFMA), offs_p, back if padded else None, T)
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


# ----------------------------------------------------------------------------- fused blocks
# The SwiGLU feed-forward block, the expert block and the routed half of an MoE layer as single
# operators: their bodies are the very functions the eager autograd functions run
# (mx_blocks.ffn_forward / ffn_backward and their grouped and routed counterparts), so a compiled
# block keeps the eager kernel sequence -- one cast of x for w1 and w3, the gate and its backward
# inside the casts, the gather, score multiply and combine of the routed tokens inside theirs,
# cached weight casts -- and equals it bit for bit.  A forward operator returns its output
# followed by a fixed number of tensors for the backward, empty where the eager function keeps
# nothing; tensors that are inputs (x, the norm weight) are kept by the autograd wrapper itself,
# since an operator's outputs may not alias its inputs.
def _empty(dev):
    return torch.empty((0,), dtype=torch.uint8, device=dev)


def _filled(saved, dev, skip=()):
    return [(_empty(dev) if (t is None or i in skip) else t) for i, t in enumerate(saved)]


def _restored(saved):
    return [(t if t.numel() else None) for t in saved]


def _block_cfg(mode: int, cache_w: bool, pad: bool = True):
    from .mx_tensor import MXFP8Config

    return MXFP8Config(scale_mode=_MODE_NAMES[mode], pad_token_groups_for_grouped_mm=pad, cache_weight_casts=cache_w)


def _pack_pair(g1, g3, dev):
    """dW1 and dW3 as ONE operator output (the two halves of one launch's output share their
    storage, and an operator's outputs may not alias each other): [2, ...] when both exist,
    [1, ...] for one, empty for none."""
    if g1 is not None and g3 is not None:
        base = g1._base
        if base is not None and base is g3._base and base.shape[0] == 2:
            return base
        return torch.stack((g1, g3))
    one = g1 if g1 is not None else g3
    return one.unsqueeze(0) if one is not None else torch.empty((0,), dtype=torch.bfloat16, device=dev)


def _unpack_pair(pack, need1: bool, need3: bool):
    if need1 and need3:
        return pack[0], pack[1]
    return (pack[0] if need1 else None), (pack[0] if need3 else None)


def _pair_shape(shape, need1: bool, need3: bool):
    n = int(need1) + int(need3)
    return (n, *shape) if n else (0,)


def _u8(shape, dev):
    return torch.empty(shape, dtype=torch.uint8, device=dev)


def _mfma(rows: int, nblk: int, dev):
    return _u8((ops.mfma_scale_bytes(rows, nblk),), dev)


_T3 = tuple[(torch.Tensor,) * 3]
_T4 = tuple[(torch.Tensor,) * 4]
_T5 = tuple[(torch.Tensor,) * 5]
_T15 = tuple[(torch.Tensor,) * 15]
_T18 = tuple[(torch.Tensor,) * 18]


@torch.library.custom_op("torchtitan_amd::mx_ffn_fwd", mutates_args=())
def mx_ffn_fwd(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor, norm_weight: torch.Tensor | None,
               eps: float, mode: int, cache_w: bool, need_dx: bool, need_dw: bool) -> _T15:
    """(y, 14 tensors for the backward) of the SwiGLU block w2(silu(w1 x) * w3 x), RMSNorm in front
    when `norm_weight` is given."""
    from . import mx_blocks

    D = x.shape[-1]
    x2 = x.reshape(-1, D)
    if x2.dtype != torch.bfloat16:
        x2 = x2.to(torch.bfloat16)
    y, saved = mx_blocks.ffn_forward(x2, None, w1, w2, w3, _block_cfg(mode, cache_w), need_dx, need_dw, norm_weight, eps)
    return (y.view(*x.shape[:-1], w2.shape[0]), *_filled(saved, x.device, skip=(11, 13)))


@mx_ffn_fwd.register_fake
def _(x, w1, w2, w3, norm_weight, eps, mode, cache_w, need_dx, need_dw):
    D, H, O = x.shape[-1], w1.shape[0], w2.shape[0]
    M = x.numel() // D
    torch._check(D % 32 == 0 and H % 32 == 0 and O % 32 == 0 and M % 32 == 0,
                 lambda: "the traced SwiGLU block needs tokens and sizes that are multiples of 32")
    dev = x.device
    s = [_empty(dev) for _ in range(14)]
    if need_dx or need_dw:
        s[0:3] = [torch.empty((2, M, H), dtype=torch.bfloat16, device=dev), _u8((H, O), dev), _mfma(H, O // 32, dev)]
    if need_dw:
        s[3:7] = [_u8((D, M), dev), _mfma(D, M // 32, dev), _u8((H, M), dev), _mfma(H, M // 32, dev)]
    if need_dx:
        s[7:11] = [_u8((D, H), dev), _mfma(D, H // 32, dev), _u8((D, H), dev), _mfma(D, H // 32, dev)]
        if norm_weight is not None:
            s[12] = torch.empty((M,), dtype=torch.float32, device=dev)
    return (x.new_empty((*x.shape[:-1], O), dtype=torch.bfloat16), *s)


@torch.library.custom_op("torchtitan_amd::mx_ffn_bwd", mutates_args=())
def mx_ffn_bwd(dy: torch.Tensor, saved: list[torch.Tensor], x: torch.Tensor | None, norm_weight: torch.Tensor | None,
               mode: int, need_x: bool, need_dw1: bool, need_dw2: bool, need_dw3: bool, need_dnw: bool) -> _T4:
    """(dx [M, in], dW1 and dW3 stacked, dW2, d norm weight) in bf16, empty where not asked for."""
    from . import mx_blocks

    s = _restored(saved)
    if norm_weight is not None:
        s[11], s[13] = x.reshape(-1, x.shape[-1]).contiguous(), norm_weight
    dy2 = dy.reshape(-1, dy.shape[-1])
    if dy2.dtype != torch.bfloat16:
        dy2 = dy2.to(torch.bfloat16)
    dx, dw1, dw2, dw3, dnw = mx_blocks.ffn_backward(dy2.contiguous(), s, _block_cfg(mode, False), need_x, need_dw1,
                                                    need_dw2, need_dw3, need_dnw)
    none = lambda: torch.empty((0,), dtype=torch.bfloat16, device=dy.device)
    return (dx if (dx is not None and need_x) else none(), _pack_pair(dw1, dw3, dy.device),
            dw2 if dw2 is not None else none(), dnw if dnw is not None else none())


@mx_ffn_bwd.register_fake
def _(dy, saved, x, norm_weight, mode, need_x, need_dw1, need_dw2, need_dw3, need_dnw):
    dev = dy.device
    bf = lambda shape, on: torch.empty(shape if on else (0,), dtype=torch.bfloat16, device=dev)
    M = dy.numel() // dy.shape[-1]
    H = saved[0].shape[2]
    D = saved[7].shape[0] if saved[7].numel() else (saved[3].shape[0] if saved[3].numel() else 0)
    O = dy.shape[-1]
    dx = bf((M, D), need_x)
    if norm_weight is not None and need_x:
        dx = torch.empty((M, D), dtype=x.dtype, device=dev)
    dnw = torch.empty(norm_weight.shape if (norm_weight is not None and need_dnw) else (0,),
                      dtype=norm_weight.dtype if norm_weight is not None else torch.bfloat16, device=dev)
    return (dx, bf(_pair_shape((H, D), need_dw1, need_dw3), True), bf((O, H), need_dw2), dnw)


def _ffn_setup(ctx, inputs, output):
    x, w1, w2, w3, norm_weight, eps, mode, cache_w, need_dx, need_dw = inputs
    ctx.normed = norm_weight is not None
    ctx.save_for_backward(*output[1:], *((x, norm_weight) if ctx.normed else ()))
    ctx.mode, ctx.x_shape = mode, x.shape
    ctx.dtypes = (x.dtype, w1.dtype, w2.dtype, w3.dtype)


def _ffn_backward(ctx, gy, *unused):
    saved = list(ctx.saved_tensors)
    x, nw = (saved[14], saved[15]) if ctx.normed else (None, None)
    need = ctx.needs_input_grad
    dx, dw13, dw2, dnw = torch.ops.torchtitan_amd.mx_ffn_bwd(gy, saved[:14], x, nw, ctx.mode, need[0], need[1],
                                                           need[2], need[3], bool(ctx.normed and need[4]))
    dw1, dw3 = _unpack_pair(dw13, need[1], need[3])
    back = lambda g, on, dt: g.to(dt) if on else None
    return (back(dx, need[0], ctx.dtypes[0]).view(ctx.x_shape) if need[0] else None, back(dw1, need[1], ctx.dtypes[1]),
            back(dw2, need[2], ctx.dtypes[2]), back(dw3, need[3], ctx.dtypes[3]),
            (dnw if (ctx.normed and need[4]) else None), None, None, None, None, None)


mx_ffn_fwd.register_autograd(_ffn_backward, setup_context=_ffn_setup)


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def mx_feed_forward_traced(x, w1, w2, w3, bias2, norm_weight=None, eps: float = 0.0):
    """The fused SwiGLU block while a graph is being traced; the weights may still be the wrapper
    subclass (the caller has switched its ``__torch_function__`` off)."""
    cfg = w2.mx_config
    need_dx = _wants_grad(x, norm_weight)
    need_dw = _wants_grad(w1, w2, w3)
    y = torch.ops.torchtitan_amd.mx_ffn_fwd(x, w1, w2, w3, norm_weight, float(eps), ops.SCALE_MODES[cfg.scale_mode],
                                            cfg.cache_weight_casts, need_dx, need_dw)[0]
    if bias2 is not None:
        y = y + bias2.to(y.dtype)
    return y


# ---- the expert block
@torch.library.custom_op("torchtitan_amd::mx_grouped_ffn_fwd", mutates_args=())
def mx_grouped_ffn_fwd(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor, offs: torch.Tensor,
                       mode: int, pad: bool, cache_w: bool, need_dx: bool, need_dw: bool) -> _T15:
    """(y [T, D] bf16, 14 tensors for the backward) of grouped_mm(silu(grouped_mm(x, w1)) * grouped_mm(x, w3), w2)."""
    from . import mx_blocks

    xb = x if x.dtype == torch.bfloat16 else x.to(torch.bfloat16)
    y, saved = mx_blocks.grouped_ffn_forward(xb, w1, w2, w3, offs, _block_cfg(mode, cache_w, pad), need_dx, need_dw)
    if saved[0] is offs:
        saved[0] = offs.clone()
    return (y, *_filled(saved, x.device))


def _grouped_ffn_sizes(T, D, H, G, pad):
    from . import mx_blocks

    order, multiple, fast = mx_blocks.grouped_layout(D, H, G)
    padded = pad or fast
    step = max(ops.BLOCK, multiple)
    Tp = -(-(T + ops.BLOCK * G) // step) * step if padded else T
    return order, padded, Tp


@mx_grouped_ffn_fwd.register_fake
def _(x, w1, w2, w3, offs, mode, pad, cache_w, need_dx, need_dw):
    T, D = x.shape
    G, H, _ = w1.shape
    torch._check(D % 32 == 0 and H % 32 == 0, lambda: "the traced expert block needs sizes that are multiples of 32")
    order, padded, Tp = _grouped_ffn_sizes(T, D, H, G, pad)
    dev = x.device
    s = [_empty(dev) for _ in range(14)]
    s[0] = torch.empty((G,), dtype=torch.int32, device=dev)
    if padded:
        s[1] = torch.empty((Tp,), dtype=torch.int64, device=dev)
        from . import mx_blocks

        fast = mx_blocks.grouped_layout(D, H, G)[2]
        s[2] = torch.empty((G,) if fast else (T,), dtype=torch.int32 if fast else torch.int64, device=dev)
    if need_dx or need_dw:
        s[3:6] = [torch.empty((2, Tp, H), dtype=torch.bfloat16, device=dev), _u8((G, H, D), dev),
                  _u8((G * ops.mfma_scale_bytes(H, D // 32),), dev)]
    if need_dw:
        s[6:10] = [_u8((D, Tp), dev), _fake_scales(D, Tp // 32, order, dev), _u8((H, Tp), dev),
                   _fake_scales(H, Tp // 32, order, dev)]
    if need_dx:
        wq = lambda: [_u8((G, D, H), dev), _u8((G * ops.mfma_scale_bytes(D, H // 32),), dev)]
        s[10:14] = wq() + wq()
    return (torch.empty((T, D), dtype=torch.bfloat16, device=dev), *s)


@torch.library.custom_op("torchtitan_amd::mx_grouped_ffn_bwd", mutates_args=())
def mx_grouped_ffn_bwd(dy: torch.Tensor, saved: list[torch.Tensor], mode: int, order: int, need_dx: bool, need_dw1: bool,
                       need_dw2: bool, need_dw3: bool) -> _T3:
    """(dx [T, D], dW1 and dW3 stacked, dW2) in bf16, empty where not asked for."""
    from . import mx_blocks

    dyb = (dy if dy.dtype == torch.bfloat16 else dy.to(torch.bfloat16)).contiguous()
    dx, dw1, dw2, dw3 = mx_blocks.grouped_ffn_backward(dyb, _restored(saved), _block_cfg(mode, False), order, need_dx,
                                                       need_dw1, need_dw2, need_dw3)
    none = lambda: torch.empty((0,), dtype=torch.bfloat16, device=dy.device)
    return (dx if dx is not None else none(), _pack_pair(dw1, dw3, dy.device), dw2 if dw2 is not None else none())


@mx_grouped_ffn_bwd.register_fake
def _(dy, saved, mode, order, need_dx, need_dw1, need_dw2, need_dw3):
    dev = dy.device
    bf = lambda shape, on: torch.empty(shape if on else (0,), dtype=torch.bfloat16, device=dev)
    T, D = dy.shape
    G, H = saved[4].shape[0], saved[4].shape[1]
    return (bf((T, D), need_dx), bf(_pair_shape((G, H, D), need_dw1, need_dw3), True), bf((G, D, H), need_dw2))


def _grouped_ffn_setup(ctx, inputs, output):
    x, w1, w2, w3, offs, mode, pad, cache_w, need_dx, need_dw = inputs
    ctx.save_for_backward(*output[1:])
    ctx.mode = mode
    ctx.order = _grouped_ffn_sizes(x.shape[0], x.shape[1], w1.shape[1], w1.shape[0], pad)[0]
    ctx.dtypes = (x.dtype, w1.dtype, w2.dtype, w3.dtype)


def _grouped_ffn_backward(ctx, gy, *unused):
    need = ctx.needs_input_grad
    dx, dw13, dw2 = torch.ops.torchtitan_amd.mx_grouped_ffn_bwd(gy, list(ctx.saved_tensors), ctx.mode, ctx.order, need[0],
                                                              need[1], need[2], need[3])
    dw1, dw3 = _unpack_pair(dw13, need[1], need[3])
    grads = (dx, dw1, dw2, dw3)
    return (*(g.to(dt) if on else None for g, dt, on in zip(grads, ctx.dtypes, need[:4])), None, None, None, None, None, None)


mx_grouped_ffn_fwd.register_autograd(_grouped_ffn_backward, setup_context=_grouped_ffn_setup)


def mx_grouped_feed_forward_traced(x, w1, w2, w3, offs):
    """The fused expert block while a graph is being traced (weights as for the dense block)."""
    cfg = w2.mx_config
    return torch.ops.torchtitan_amd.mx_grouped_ffn_fwd(
        x, w1, w2, w3, offs.to(torch.int32), ops.SCALE_MODES[cfg.scale_mode], cfg.pad_token_groups_for_grouped_mm,
        cfg.cache_weight_casts, _wants_grad(x), _wants_grad(w1, w2, w3))[0]


# ---- the routed half of an MoE layer
@torch.library.custom_op("torchtitan_amd::mx_routed_experts_fwd", mutates_args=())
def mx_routed_experts_fwd(x: torch.Tensor, top_scores: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor,
                          tok_sorted: torch.Tensor, counts: torch.Tensor, score_before: bool, mode: int, cache_w: bool,
                          need_dx: bool, need_ds: bool, need_dw: bool) -> _T18:
    """(out [T, D] bf16, 17 tensors for the backward) of the routed experts with gather, score
    multiply and combine inside the cast / combine kernels."""
    from . import mx_blocks

    xb = (x if x.dtype == torch.bfloat16 else x.to(torch.bfloat16)).contiguous()
    out, saved = mx_blocks.routed_forward(xb, top_scores, w1, w2, w3, tok_sorted, counts, score_before,
                                          _block_cfg(mode, cache_w), need_dx, need_ds, need_dw)
    if saved[4].data_ptr() == top_scores.data_ptr():
        saved[4] = saved[4].clone()
    skip = (16,) if score_before else ()  # x itself: kept by the autograd wrapper
    return (out, *_filled(saved, x.device, skip=skip))


@mx_routed_experts_fwd.register_fake
def _(x, top_scores, w1, w2, w3, tok_sorted, counts, score_before, mode, cache_w, need_dx, need_ds, need_dw):
    from . import mx_blocks

    T, D = x.shape
    k = top_scores.shape[1]
    G, H, _ = w1.shape
    torch._check(D % 32 == 0 and H % 32 == 0, lambda: "the traced routed experts need sizes that are multiples of 32")
    order, multiple, _ = mx_blocks.grouped_layout(D, H, G)
    step = max(ops.BLOCK, multiple)
    Tp = -(-(T * k + ops.BLOCK * G) // step) * step
    dev = x.device
    s = [_empty(dev) for _ in range(17)]
    s[0] = torch.empty((G,), dtype=torch.int32, device=dev)
    s[1] = torch.empty((Tp,), dtype=torch.int64, device=dev)
    s[2] = torch.empty((Tp,), dtype=torch.float32, device=dev)
    s[3] = torch.empty((T, k), dtype=torch.int64, device=dev)
    s[4] = torch.empty((T, k), dtype=torch.float32, device=dev)
    if need_dx or need_ds or need_dw:
        s[5:8] = [torch.empty((2, Tp, H), dtype=torch.bfloat16, device=dev), _u8((G, H, D), dev),
                  _u8((G * ops.mfma_scale_bytes(H, D // 32),), dev)]
    if need_dw:
        s[8:12] = [_u8((D, Tp), dev), _fake_scales(D, Tp // 32, order, dev), _u8((H, Tp), dev),
                   _fake_scales(H, Tp // 32, order, dev)]
    if need_dx or need_ds:
        wq = lambda: [_u8((G, D, H), dev), _u8((G * ops.mfma_scale_bytes(D, H // 32),), dev)]
        s[12:16] = wq() + wq()
    if need_ds and not score_before:
        s[16] = torch.empty((Tp, D), dtype=torch.bfloat16, device=dev)
    return (torch.empty((T, D), dtype=torch.bfloat16, device=dev), *s)


@torch.library.custom_op("torchtitan_amd::mx_routed_experts_bwd", mutates_args=())
def mx_routed_experts_bwd(dout: torch.Tensor, saved: list[torch.Tensor], x: torch.Tensor | None, mode: int, order: int,
                          score_before: bool, need_dx: bool, need_ds: bool, need_dw1: bool, need_dw2: bool,
                          need_dw3: bool) -> _T4:
    """(dx [T, D] bf16, d scores [T, k] float32, dW1 and dW3 stacked, dW2 bf16), empty where not
    asked for."""
    from . import mx_blocks

    s = _restored(saved)
    if x is not None:
        s[16] = (x if x.dtype == torch.bfloat16 else x.to(torch.bfloat16)).contiguous()
    dob = (dout if dout.dtype == torch.bfloat16 else dout.to(torch.bfloat16)).contiguous()
    dx, ds, dw1, dw2, dw3 = mx_blocks.routed_backward(dob, s, _block_cfg(mode, False), order, score_before, need_dx,
                                                      need_ds, need_dw1, need_dw2, need_dw3)
    none = lambda dt=torch.bfloat16: torch.empty((0,), dtype=dt, device=dout.device)
    return (dx if dx is not None else none(), ds if ds is not None else none(torch.float32),
            _pack_pair(dw1, dw3, dout.device), dw2 if dw2 is not None else none())


@mx_routed_experts_bwd.register_fake
def _(dout, saved, x, mode, order, score_before, need_dx, need_ds, need_dw1, need_dw2, need_dw3):
    dev = dout.device
    mk = lambda shape, on, dt=torch.bfloat16: torch.empty(shape if on else (0,), dtype=dt, device=dev)
    T, D = dout.shape
    k = saved[3].shape[1]
    G, H = saved[6].shape[0], saved[6].shape[1]
    return (mk((T, D), need_dx), mk((T, k), need_ds, torch.float32), mk(_pair_shape((G, H, D), need_dw1, need_dw3), True),
            mk((G, D, H), need_dw2))


def _routed_setup(ctx, inputs, output):
    x, top_scores, w1, w2, w3, tok_sorted, counts, score_before, mode, cache_w, need_dx, need_ds, need_dw = inputs
    ctx.keep_x = bool(score_before and need_ds)
    ctx.save_for_backward(*output[1:], *((x,) if ctx.keep_x else ()))
    from . import mx_blocks

    ctx.mode, ctx.score_before = mode, score_before
    ctx.order = mx_blocks.grouped_layout(x.shape[1], w1.shape[1], w1.shape[0])[0]
    ctx.dtypes = (x.dtype, top_scores.dtype, w1.dtype, w2.dtype, w3.dtype)


def _routed_backward(ctx, gout, *unused):
    saved = list(ctx.saved_tensors)
    x = saved[17] if ctx.keep_x else None
    need = ctx.needs_input_grad
    dx, ds, dw13, dw2 = torch.ops.torchtitan_amd.mx_routed_experts_bwd(gout, saved[:17], x, ctx.mode, ctx.order,
                                                                     ctx.score_before, need[0], need[1], need[2], need[3],
                                                                     need[4])
    dw1, dw3 = _unpack_pair(dw13, need[2], need[4])
    grads = (dx, ds, dw1, dw2, dw3)
    return (*(g.to(dt) if on else None for g, dt, on in zip(grads, ctx.dtypes, need[:5])),
            None, None, None, None, None, None, None, None)


mx_routed_experts_fwd.register_autograd(_routed_backward, setup_context=_routed_setup)


def mx_routed_experts_traced(x, top_scores, w1, w2, w3, tok_sorted, counts, score_before: bool):
    """The fused routed half of an MoE layer while a graph is being traced."""
    cfg = w2.mx_config
    return torch.ops.torchtitan_amd.mx_routed_experts_fwd(
        x, top_scores, w1, w2, w3, tok_sorted, counts, bool(score_before), ops.SCALE_MODES[cfg.scale_mode],
        cfg.cache_weight_casts, _wants_grad(x), _wants_grad(top_scores), _wants_grad(w1, w2, w3))[0]
