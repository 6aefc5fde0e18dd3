"""Weight wrapper that re-routes ``F.linear`` and ``torch._grouped_mm`` to the MXFP8 kernels.

After conversion a target weight is still an ordinary trainable high-precision parameter
(optimizer, ``init_weights``, ``to_empty`` and checkpointing keep working on it), but it is an
instance of ``MXFP8TrainingWeight``; its ``__torch_function__`` sends the two GEMM entry points
to autograd functions that quantize dynamically and call the HIP library in forward and
backward.  This is the role the reference gives to the external tensor subclass installed by
its converter (torchtitan/components/quantization/mx.py:27-31,93-96,119-125).

Passes of one linear with W [N, K], X [M, K], dY [M, N]  (every GEMM is "NT"):
    forward  Y  = cast_dim0(X)  x cast_dim0(W)        contraction K
    dgrad    dX = cast_dim0(dY) x cast_dim1(W)        contraction N
    wgrad    dW = cast_dim1(dY) x cast_dim1(X)        contraction M
X and W are read once in forward (fused row+column cast) and their column-wise forms are what
is saved for backward; dY is read once in backward.
"""
from __future__ import annotations

import weakref

import torch
import torch.nn.functional as F

from . import ops
from .ops import MX_SCALES_MFMA, MX_SCALES_ROWMAJOR, MXData


class MXFP8Config:
    """Per-weight recipe: scale mode and whether grouped GEMMs pad token groups to 32."""

    __slots__ = ("scale_mode", "pad_token_groups_for_grouped_mm", "fuse_swiglu_cast", "cache_weight_casts",
                 "fuse_rmsnorm_cast")

    def __init__(self, scale_mode: str = "rceil", pad_token_groups_for_grouped_mm: bool = True,
                 fuse_swiglu_cast: bool = True, cache_weight_casts: bool = False,
                 fuse_rmsnorm_cast: bool = False):
        if scale_mode not in ops.SCALE_MODES:
            raise ValueError(f"unknown scale mode {scale_mode!r}")
        self.scale_mode = scale_mode
        self.pad_token_groups_for_grouped_mm = pad_token_groups_for_grouped_mm
        self.fuse_swiglu_cast = fuse_swiglu_cast
        self.cache_weight_casts = cache_weight_casts
        self.fuse_rmsnorm_cast = fuse_rmsnorm_cast

    def __repr__(self):
        return (f"MXFP8Config(scale_mode={self.scale_mode!r}, "
                f"pad_token_groups_for_grouped_mm={self.pad_token_groups_for_grouped_mm})")


# ----------------------------------------------------------------------------- cast reuse
class _ActivationCastCache:
    """Remembers the fused cast of the last activation tensor.

    w1(x) and w3(x) of a SwiGLU block, or wq/wk/wv of attention, receive the same tensor object;
    the second and third linear reuse the codes instead of re-reading x.  The entry is keyed on
    object identity, the tensor's version counter and its address, and holds only a weak
    reference to the activation.

    What keeps a hit from being stale: an entry lives for one forward at most.  It is dropped at
    the start of every backward of a converted linear, whenever the stream's graph-capture state
    changes (an entry made by an eager warm-up is never reused under capture, so the cast is
    always recorded into the graph, and an entry made under capture is never reused by eager
    code), and by `clear_cast_cache()`.  Writes through this package's `out=` arguments bump the
    destination's version counter.  A caller that overwrites an activation behind autograd's back
    (`.data`, a foreign kernel) between two forwards without a backward in between must call
    `clear_cast_cache()`.
    """

    def __init__(self):
        self._ref = None
        self._key = None
        self._value = None
        self._capturing = False

    def _sync_capture_state(self):
        capturing = torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()
        if capturing != self._capturing:
            self.clear()
            self._capturing = capturing

    def get(self, x: torch.Tensor, mode: str):
        self._sync_capture_state()
        if self._ref is not None and self._ref() is x and self._key == (x._version, mode, x.data_ptr()):
            return self._value
        return None

    def put(self, x: torch.Tensor, mode: str, value):
        self._sync_capture_state()
        self._ref = weakref.ref(x)
        self._key = (x._version, mode, x.data_ptr())
        self._value = value

    def clear(self):
        self._ref = self._key = self._value = None


_cast_cache = _ActivationCastCache()


def clear_cast_cache() -> None:
    """Forget the remembered activation cast (see `_ActivationCastCache`)."""
    _cast_cache.clear()


def _cast_activation(x2: torch.Tensor, src: torch.Tensor, mode: str, need_cols: bool, pitch_pad: int = 0):
    """(row-wise, column-wise or None) MXFP8 forms of the 2-D bf16 activation `x2`.  `pitch_pad`:
    see `ops.to_mx_dim0_dim1`; callers that feed anything but `ops.mx_gemm_nt` leave it 0."""
    key = (mode, pitch_pad)
    hit = _cast_cache.get(src, key)
    if hit is not None and (hit[1] is not None or not need_cols):
        return hit
    if need_cols and x2.shape[0] % ops.BLOCK == 0:
        rows, cols = ops.to_mx_dim0_dim1(x2, mode, MX_SCALES_MFMA, pitch_pad)
    else:
        rows, cols = ops.to_mx_dim0(x2, mode, MX_SCALES_MFMA), None
    _cast_cache.put(src, key, (rows, cols))
    return rows, cols


# ----------------------------------------------------------------------------- weight casts
class _WeightCastCache:
    """MXFP8 forms of weights that have not changed since they were cast.

    A weight changes once per optimizer step but is cast in every forward; with gradient
    accumulation, several forwards per step, or a hand-over of the weights in MXFP8 form, the
    casts after the first are repeats.  An entry is keyed on the weight's memory (address, shape,
    strides) and valid while that storage is alive and its version counter is unchanged: every
    in-place update (optimizer step, ``copy_``, init) invalidates it.  Off unless the converter
    is built with ``cache_weight_casts=True``; holds 2 bytes per weight element."""

    def __init__(self):
        self._entries = {}

    @staticmethod
    def _key(w: torch.Tensor, mode: str):
        return (w.data_ptr(), tuple(w.shape), tuple(w.stride()), w.dtype, mode)

    def get(self, w: torch.Tensor, mode: str):
        e = self._entries.get(self._key(w, mode))
        if e is None:
            return None
        ref, version, rows, cols = e
        if ref.expired() or version != w._version:
            return None
        return rows, cols

    def put(self, w: torch.Tensor, mode: str, rows: MXData, cols):
        from torch.multiprocessing.reductions import StorageWeakRef

        dead = [k for k, e in self._entries.items() if e[0].expired()]
        for k in dead:
            del self._entries[k]
        self._entries[self._key(w, mode)] = (StorageWeakRef(w.untyped_storage()), w._version, rows, cols)

    def clear(self):
        self._entries.clear()

    def __len__(self):
        return len(self._entries)


_weight_cache = _WeightCastCache()


def _cast_weight(w: torch.Tensor, mode: str, need_cols: bool, cfg: MXFP8Config, pitch_pad: int = 0):
    """(row-wise, column-wise or None) MXFP8 forms of a weight [N, K] or stacked [G, N, K], MFMA
    scale order.  The column-wise form exists when asked for and N is a multiple of 32.
    `pitch_pad` (2-D weights, both forms asked for): see `ops.to_mx_dim0_dim1`."""
    cached = cfg.cache_weight_casts
    mode_key = mode
    if pitch_pad:
        mode = (mode, pitch_pad)  # the cache keeps padded and dense casts apart
    if cached:
        hit = _weight_cache.get(w, mode)
        if hit is not None and (hit[1] is not None or not need_cols or w.shape[-2] % ops.BLOCK):
            return hit
        need_cols = True  # cast once in full, whoever asks first
    key, mode = mode, mode_key
    wb = (w if w.dtype == torch.bfloat16 else w.to(torch.bfloat16)).contiguous()
    both = need_cols and wb.shape[-2] % ops.BLOCK == 0
    if wb.dim() == 3:
        q = ops.to_mx_dim0_dim1_batched(wb, mode, MX_SCALES_MFMA) if both else (_cast_w_rows(wb, mode), None)
    else:
        q = (ops.to_mx_dim0_dim1(wb, mode, MX_SCALES_MFMA, pitch_pad) if both
             else (ops.to_mx_dim0(wb, mode, MX_SCALES_MFMA), None))
    if cached:
        _weight_cache.put(w, key, q[0], q[1])
    return q


# ----------------------------------------------------------------------------- dense linear
class _MXLinear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, cfg: MXFP8Config):
        mode = cfg.scale_mode
        K = x.shape[-1]
        N = weight.shape[0]
        x2 = x.reshape(-1, K)
        if x2.dtype != torch.bfloat16:
            x2 = x2.to(torch.bfloat16)
        w = weight if weight.dtype == torch.bfloat16 else weight.to(torch.bfloat16)
        needs_bwd = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        M = x2.shape[0]
        # operands of mx_gemm_nt only: their rows may lie further apart than they are long (not with
        # cached weight casts, which the fused blocks and the hand-over share in their dense form)
        pad = 0 if cfg.cache_weight_casts else ops.CODE_PITCH_PAD
        xq0, xq1 = _cast_activation(x2, x, mode, need_cols=ctx.needs_input_grad[1], pitch_pad=pad)
        wq0, wq1 = _cast_weight(weight, mode, needs_bwd and ctx.needs_input_grad[0], cfg, pitch_pad=pad)
        y = ops.mx_gemm_nt(xq0, wq0)
        ctx.cfg = cfg
        ctx.x_shape = x.shape
        ctx.x_dtype = x.dtype
        ctx.w_dtype = weight.dtype
        ctx.have_xq1 = xq1 is not None
        ctx.have_wq1 = wq1 is not None
        saved = []
        if ctx.needs_input_grad[1]:
            saved += [xq1.codes, xq1.scales] if xq1 is not None else [x2]
        if ctx.needs_input_grad[0]:
            saved += [wq1.codes, wq1.scales] if wq1 is not None else [w]
        ctx.save_for_backward(*saved)
        return y.view(*x.shape[:-1], N)

    @staticmethod
    def backward(ctx, dy):
        _cast_cache.clear()  # the forward whose sibling linears shared a cast is over
        mode = ctx.cfg.scale_mode
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        saved = list(ctx.saved_tensors)
        N = dy.shape[-1]
        dy2 = dy.reshape(-1, N)
        if dy2.dtype != torch.bfloat16:
            dy2 = dy2.to(torch.bfloat16)
        dy2 = dy2.contiguous()
        M = dy2.shape[0]
        xq1 = wq1 = None
        if need_dw:
            if ctx.have_xq1:
                xq1 = MXData(saved.pop(0), saved.pop(0), MX_SCALES_MFMA)
            else:  # M not a multiple of 32: pad the token dim with zero rows for the column cast
                xq1 = _cast_cols_padded(saved.pop(0), mode)
        if need_dx:
            if ctx.have_wq1:
                wq1 = MXData(saved.pop(0), saved.pop(0), MX_SCALES_MFMA)
            else:
                wq1 = _cast_cols_padded(saved.pop(0), mode)
        dyq0 = dyq1 = None
        if need_dx and need_dw and M % ops.BLOCK == 0 and N % ops.BLOCK == 0:
            dyq0, dyq1 = ops.to_mx_dim0_dim1(dy2, mode, MX_SCALES_MFMA,
                                             0 if ctx.cfg.cache_weight_casts else ops.CODE_PITCH_PAD)
        else:
            if need_dx:
                dyq0 = _cast_rows_padded(dy2, mode)
            if need_dw:
                dyq1 = _cast_cols_padded(dy2, mode)
        dx = dw = None
        if need_dx:
            dx = ops.mx_gemm_nt(dyq0, wq1).view(ctx.x_shape)
            if dx.dtype != ctx.x_dtype:
                dx = dx.to(ctx.x_dtype)
        if need_dw:
            dw = ops.mx_gemm_nt(dyq1, xq1)
            if dw.dtype != ctx.w_dtype:
                dw = dw.to(ctx.w_dtype)
        return dx, dw, None


def _cast_cols_padded(t: torch.Tensor, mode: str) -> MXData:
    """Column-wise cast of t [R, C]; R is zero-padded up to a multiple of 32 (zeros add nothing
    to a contraction over R)."""
    R = t.shape[0]
    pad = -R % ops.BLOCK
    if pad:
        t = torch.cat((t, t.new_zeros((pad, t.shape[1]))), dim=0)
    return ops.to_mx_dim1(t.contiguous(), mode, MX_SCALES_MFMA)


def _cast_rows_padded(t: torch.Tensor, mode: str) -> MXData:
    """Row-wise cast of t [R, C]; C is zero-padded up to a multiple of 32."""
    C = t.shape[1]
    pad = -C % ops.BLOCK
    if pad:
        t = torch.cat((t, t.new_zeros((t.shape[0], pad))), dim=1)
    return ops.to_mx_dim0(t.contiguous(), mode, MX_SCALES_MFMA)


def mx_linear(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, cfg: MXFP8Config):
    """``F.linear`` with the matmul in MXFP8; the bias add stays in high precision."""
    if x.shape[-1] % ops.BLOCK:
        raise ValueError(f"MXFP8 linear needs in_features % 32 == 0, got {x.shape[-1]}")
    out_dtype = x.dtype
    if torch.is_autocast_enabled(x.device.type):
        out_dtype = torch.get_autocast_dtype(x.device.type)
    y = _MXLinear.apply(x, weight, cfg)
    if y.dtype != out_dtype:
        y = y.to(out_dtype)
    if bias is not None:
        y = y + bias.to(y.dtype)
    return y


# ----------------------------------------------------------------------------- grouped GEMM
def _pad_plan(offs: torch.Tensor, T: int, align: int = 32, length_multiple: int = 1, direct: bool = False):
    """Device-side plan that moves rows of variable-size groups into `align`-aligned groups.

    Returns (gather indices into [x; 0-row] for the padded layout, padded inclusive offsets,
    the way back).  The way back is, for every original row, its row in the padded layout or the
    index of an appended zero row (int64 [T]: a gather) -- or, with `direct`, a copy of the
    unpadded group ends (int32 [G]) for a grouped GEMM that writes the unpadded rows itself.
    No host synchronisation: the padded length is the static bound round_up(T + align G, align),
    rounded up further to `length_multiple` (a multiple of align) when one is given.
    """
    G = offs.numel()
    sizes = torch.diff(offs, prepend=offs.new_zeros(1))
    step = max(align, length_multiple)
    max_len = -(-(T + align * G) // step) * step
    perm, _, m_offsets = ops.group_offsets_pad(sizes, G, 1, max_len, align)
    if direct:
        return perm, m_offsets, offs.to(torch.int32).clone()
    back = torch.full((T + 1,), max_len, dtype=torch.int64, device=offs.device)
    back[perm] = torch.arange(max_len, device=offs.device)  # perm == -1 writes the spare slot T
    return perm, m_offsets, back[:T]


def _cast_into_groups(t: torch.Tensor, perm, mode: str, order: int, want_cols: bool):
    """(row-wise, column-wise or None) casts of `t` moved into its padded group layout: the
    gather by `perm` happens inside the cast kernel (padding slots read as zero rows)."""
    if perm is not None:
        return ops.to_mx_rows_gathered(t, perm, mode, order, want_cols)
    if want_cols:
        return ops.to_mx_dim0_dim1(t, mode, order)
    return ops.to_mx_dim0(t, mode, order), None


def _grouped_2d3d_padded(a: MXData, b: MXData, offs_p: torch.Tensor, back, out_rows: int,
                         a2: MXData | None = None, b2: MXData | None = None):
    """Grouped GEMM (with a2, b2: the sum of two) in the padded layout, result in the original
    row order [out_rows, N]; `back` as `_pad_plan` returns it (None: nothing was padded).  On
    the gather path one spare zero row behind the GEMM's output serves rows that belong to no
    group."""
    Tp, N = a.codes.shape[0], b.codes.shape[1]
    two = a2 is not None
    if back is not None and back.dtype == torch.int32:  # the GEMM leaves the padding out itself
        return ops.mx_grouped_gemm_2d3d_rows_out(a, b, offs_p, back, out_rows, a2, b2)
    if back is None:
        return ops.mx_grouped_gemm_2d3d_pair(a, b, a2, b2, offs_p) if two else ops.mx_grouped_gemm_2d3d(a, b, offs_p)
    if ops._watched() and not two:  # the dispatcher form of the GEMM allocates its own output
        y = ops.mx_grouped_gemm_2d3d(a, b, offs_p)
        return torch.cat((y, y.new_zeros(1, N)))[back]
    buf = torch.empty((Tp + 1, N), dtype=torch.bfloat16, device=a.codes.device)
    buf[Tp].zero_()
    if two:
        ops.mx_grouped_gemm_2d3d_pair(a, b, a2, b2, offs_p, buf[:Tp])
    else:
        ops.mx_grouped_gemm_2d3d(a, b, offs_p, buf[:Tp])
    return buf[back]


class _MXGroupedMM(torch.autograd.Function):
    """out[rows of g] = x[rows of g] @ w[g]^T with w [G, N, K]; offs = inclusive cumsum, int32."""

    @staticmethod
    def forward(ctx, x, weight, offs, cfg: MXFP8Config):
        mode = cfg.scale_mode
        T, K = x.shape
        G, N, _ = weight.shape
        xb = x if x.dtype == torch.bfloat16 else x.to(torch.bfloat16)
        w = weight if weight.dtype == torch.bfloat16 else weight.to(torch.bfloat16)
        w = w.contiguous()
        plan = None
        # Groups are padded to the 32 rows the format needs; the persistent kernel takes them as
        # they are (scales in MFMA order, the token axis rounded up to whole 128-deep blocks).
        fast = K % 128 == 0 and N % 128 == 0 and G <= ops.FAST_MAX_GROUPS
        order = MX_SCALES_MFMA if fast else MX_SCALES_ROWMAJOR
        perm = back = None
        if cfg.pad_token_groups_for_grouped_mm or fast:
            plan = _pad_plan(offs, T, ops.BLOCK, ops.FAST_LENGTH_MULTIPLE if fast else 1, direct=fast)
            perm, offs_p, back = plan
        else:
            offs_p = offs
            if T % ops.BLOCK:
                raise ValueError("without padding the token dimension must be a multiple of 32")
        xb = xb.contiguous()
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        xq0, xq1 = _cast_into_groups(xb, perm, mode, order, need_dw)
        wq0, wq1 = _cast_weight(weight, mode, need_dx, cfg)
        y = _grouped_2d3d_padded(xq0, wq0, offs_p, back, T)
        ctx.cfg = cfg
        ctx.dims = (T, K, N, G)
        ctx.dtypes = (x.dtype, weight.dtype)
        ctx.padded = plan is not None
        ctx.order = order
        saved = [offs_p]
        if plan is not None:
            saved += [plan[0], plan[2]]
        if need_dw:
            saved += [xq1.codes, xq1.scales]
        if need_dx:
            ctx.have_wq1 = wq1 is not None
            saved += [wq1.codes, wq1.scales] if wq1 is not None else [w]
        ctx.save_for_backward(*saved)
        return y

    @staticmethod
    def backward(ctx, dy):
        mode = ctx.cfg.scale_mode
        T, K, N, G = ctx.dims
        need_dx, need_dw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        saved = list(ctx.saved_tensors)
        offs_p = saved.pop(0)
        dyb = (dy if dy.dtype == torch.bfloat16 else dy.to(torch.bfloat16)).contiguous()
        perm = back = None
        if ctx.padded:
            perm, back = saved.pop(0), saved.pop(0)
        dx = dw = None
        if need_dw:
            xq1 = MXData(saved.pop(0), saved.pop(0), ctx.order)
        if ctx.padded or (need_dx and need_dw and N % ops.BLOCK == 0):
            dyq0, dyq1 = _cast_into_groups(dyb, perm, mode, ctx.order, need_dw)
        else:
            dyq0 = ops.to_mx_dim0(dyb, mode, ctx.order) if need_dx else None
            dyq1 = ops.to_mx_dim1(dyb, mode, ctx.order) if need_dw else None
        if need_dx:
            if ctx.have_wq1:
                wq1 = MXData(saved.pop(0), saved.pop(0), MX_SCALES_MFMA)
            else:
                wq1 = ops.to_mx_dim1_batched(saved.pop(0), mode, MX_SCALES_MFMA)
            dx = _grouped_2d3d_padded(dyq0, wq1, offs_p, back, T)
            if dx.dtype != ctx.dtypes[0]:
                dx = dx.to(ctx.dtypes[0])
        if need_dw:
            dw = ops.mx_grouped_gemm_2d2d(dyq1, xq1, offs_p)
            if dw.dtype != ctx.dtypes[1]:
                dw = dw.to(ctx.dtypes[1])
        return dx, dw, None, None


def _cast_w_rows(w: torch.Tensor, mode: str) -> MXData:
    """Row-wise cast of stacked matrices w [G, N, K] with one MFMA-order scale block each."""
    return ops.to_mx_dim0_batched(w, mode, MX_SCALES_MFMA)


def mx_grouped_mm(x: torch.Tensor, w_t: torch.Tensor, offs: torch.Tensor, cfg: MXFP8Config):
    """``torch._grouped_mm(x, w_t, offs=offs)`` for x [T, K], w_t [G, K, N] = weight^T."""
    if x.dim() != 2 or w_t.dim() != 3 or offs is None:
        raise NotImplementedError("MXFP8 grouped_mm supports the 2D x 3D form with offsets only")
    weight = w_t.transpose(-2, -1)  # back to the parameter's [G, N, K] layout
    if x.shape[-1] % ops.BLOCK:
        raise ValueError(f"MXFP8 grouped_mm needs K % 32 == 0, got {x.shape[-1]}")
    return _MXGroupedMM.apply(x, weight, offs.to(torch.int32), cfg)


def grouped_mm(x: torch.Tensor, w_t: torch.Tensor, offs: torch.Tensor):
    """``torch._grouped_mm(x, w_t, offs=offs)`` that reaches a converted weight in a traced graph
    too.  Eagerly the weight's ``__torch_function__`` sees ``torch._grouped_mm``; Dynamo offers it
    only the functions ``torch.overrides.get_overridable_functions()`` lists, which leaves out
    underscore names, so a traced ``torch._grouped_mm`` on a converted weight would run in bf16
    without a word.  Code that may be compiled calls this instead."""
    if (torch.compiler.is_compiling() and isinstance(w_t, MXFP8TrainingWeight)
            and not isinstance(x, MXFP8TrainingWeight)):
        from .compiled import mx_grouped_mm_traced

        cfg = w_t.mx_config
        with torch._C.DisableTorchFunctionSubclass():
            return mx_grouped_mm_traced(x, w_t, offs, cfg.scale_mode, cfg.pad_token_groups_for_grouped_mm)
    return torch._grouped_mm(x, w_t, offs=offs)


# ----------------------------------------------------------------------------- the wrapper
_LINEAR_FUNCS = {F.linear}
_GROUPED_FUNCS = {torch._grouped_mm}


def _unwrap(t):
    return t.as_subclass(torch.Tensor) if isinstance(t, MXFP8TrainingWeight) else t


class MXFP8TrainingWeight(torch.Tensor):
    """A high-precision weight whose GEMMs run in MXFP8.

    Shares storage with the tensor it was made from (like ``nn.Parameter``), so in-place
    initialisation and optimizer updates act on the real weight.  Every op other than
    ``F.linear`` / ``torch._grouped_mm`` behaves as for a plain tensor, and results that are
    views or casts of the weight stay wrapped so that ``w.bfloat16().transpose(-2, -1)`` still
    reaches the grouped kernel.
    """

    mx_config: MXFP8Config = MXFP8Config()

    @staticmethod
    def __new__(cls, data: torch.Tensor, config: MXFP8Config | None = None):
        t = torch.Tensor._make_subclass(cls, data, data.requires_grad)
        t.mx_config = config or MXFP8Config()
        return t

    def __repr__(self):
        return f"MXFP8TrainingWeight({self.as_subclass(torch.Tensor)!r}, config={self.mx_config!r})"

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        if func in _LINEAR_FUNCS:
            x = args[0]
            w = args[1] if len(args) > 1 else kwargs["weight"]
            b = args[2] if len(args) > 2 else kwargs.get("bias")
            if isinstance(w, cls) and not isinstance(x, cls):
                if torch.compiler.is_compiling():
                    # a tracer cannot follow the eager path's library calls: the linear enters
                    # the graph as one opaque operator (torchtitan_amd/compiled.py)
                    from .compiled import mx_linear_traced

                    with torch._C.DisableTorchFunctionSubclass():
                        return mx_linear_traced(x, w, b, w.mx_config.scale_mode, w.mx_config.cache_weight_casts)
                return mx_linear(x, _unwrap(w), _unwrap(b), w.mx_config)
        elif func in _GROUPED_FUNCS:
            a, b = args[0], args[1]
            offs = kwargs.get("offs", args[2] if len(args) > 2 else None)
            if isinstance(b, cls) and not isinstance(a, cls):
                if torch.compiler.is_compiling():  # as for the linear: one opaque operator
                    from .compiled import mx_grouped_mm_traced

                    with torch._C.DisableTorchFunctionSubclass():
                        return mx_grouped_mm_traced(a, b, offs, b.mx_config.scale_mode,
                                                    b.mx_config.pad_token_groups_for_grouped_mm)
                return mx_grouped_mm(a, _unwrap(b), offs, b.mx_config)
        cfg = next((a.mx_config for a in _flatten(args) if isinstance(a, cls)), None)
        with torch._C.DisableTorchFunctionSubclass():
            out = func(*args, **kwargs)
        return _rewrap(out, cls, cfg, func)

    # pickling: the plain tensor plus the config (and whether it was a Parameter)
    def __reduce_ex__(self, proto):
        plain = self.as_subclass(torch.Tensor)
        if getattr(self, "_is_param", False):
            return (_rebuild_parameter, (plain.detach(), self.mx_config, self.requires_grad))
        return (MXFP8TrainingWeight, (plain, self.mx_config))

    def __deepcopy__(self, memo):
        """An independent copy that is still a converted weight (and still a Parameter if this
        one is): what ``copy.deepcopy(model)`` needs, e.g. when a trainer clones a converted model
        per pipeline stage."""
        if id(self) in memo:
            return memo[id(self)]
        data = self.as_subclass(torch.Tensor).detach().clone(memory_format=torch.preserve_format)
        out = MXFP8TrainingWeight(data, self.mx_config)
        if getattr(self, "_is_param", False):
            out = _as_parameter(data, self.mx_config, self.requires_grad)
        else:
            out.requires_grad_(self.requires_grad)
        memo[id(self)] = out
        return out


def _as_parameter(data: torch.Tensor, cfg: MXFP8Config, requires_grad: bool) -> "MXFP8TrainingWeight":
    """A converted weight that is an ``nn.Parameter`` (``isinstance`` holds through the
    ``_is_param`` mark ``nn.Parameter`` itself puts on tensor subclasses), sharing `data`'s
    storage.  Built directly rather than through ``nn.Parameter(wrapper)``: that detaches the
    wrapper, and the result is a view whose base keeps the dtype and device of conversion time
    when ``module.to(...)`` later swaps the parameter's data -- a tracer that checks a tensor's
    base against its fake twin then refuses the parameter."""
    t = torch.Tensor._make_subclass(MXFP8TrainingWeight, data, requires_grad)
    t.mx_config = cfg
    t._is_param = True
    return t


def _rebuild_parameter(data: torch.Tensor, cfg: MXFP8Config, requires_grad: bool):
    return _as_parameter(data, cfg, requires_grad)


# views, casts, detach and clone of a weight are still that weight, and so is the storage that
# `Module.to_empty` gives a meta-device parameter (torch.empty_like); zeros_like and the other
# factory functions (optimizer state) make plain tensors
_KEEP_WRAPPED = {
    torch.Tensor.transpose, torch.Tensor.t, torch.Tensor.bfloat16, torch.Tensor.to,
    torch.Tensor.detach, torch.Tensor.requires_grad_, torch.Tensor.contiguous,
    torch.Tensor.view, torch.Tensor.reshape, torch.Tensor.float, torch.Tensor.half,
    torch.transpose, torch.empty_like, torch.Tensor.clone, torch.clone,
    torch.Tensor.cuda, torch.Tensor.cpu, torch.Tensor.type,
}


def _flatten(args):
    for a in args:
        if isinstance(a, (list, tuple)):
            yield from _flatten(a)
        else:
            yield a


def _rewrap(out, cls, cfg, func):
    """Results of view / cast / clone style ops on a wrapped weight stay wrapped; in-place ops
    return their (already wrapped) input; everything else is a plain tensor."""
    if cfg is None or func not in _KEEP_WRAPPED:
        return out
    if isinstance(out, torch.Tensor) and not isinstance(out, cls):
        wrapped = out.as_subclass(cls)
        wrapped.mx_config = cfg
        return wrapped
    return out


def wrap_parameter(param: torch.nn.Parameter, cfg: MXFP8Config) -> torch.nn.Parameter:
    """A Parameter of type MXFP8TrainingWeight sharing `param`'s storage."""
    if isinstance(param.data, MXFP8TrainingWeight) or isinstance(param, MXFP8TrainingWeight):
        return param
    return _as_parameter(param.data, cfg, param.requires_grad)
