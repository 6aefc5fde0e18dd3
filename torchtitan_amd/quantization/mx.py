"""``MXFP8Converter``: the model-converter plugin that switches target linears and 3-D expert
parameters to MXFP8 GEMMs on MI355X.

Same surface as the reference's converter (torchtitan/components/quantization/mx.py:26-140):
``Config(recipe_name, fqns, pad_token_groups_for_grouped_mm)``, ``_quantization_type = "mxfp8"``,
constructor kwargs ``parallel_dims`` and ``model_compile_enabled``, ``convert(model)`` mutating in
place, ``post_optimizer_hook`` a no-op.  Where the reference hands the work to an external
library and asserts an SM100 GPU, this converter wraps the weights in ``MXFP8TrainingWeight``
(backed by the in-tree HIP library) and asserts a gfx950 GPU.
"""
from __future__ import annotations

import logging
from dataclasses import dataclass, field
from functools import partial
from typing import Any, ClassVar, Literal

import torch
import torch.nn as nn

from .. import _lib
from ..modules.linear import Linear
from ..mx_tensor import MXFP8Config, MXFP8TrainingWeight, _cast_weight, wrap_parameter
from . import QuantizationConverter
from .module_utils import capture_module_attrs, inject_module_protocol, verify_module_protocol
from .utils import module_filter_fn

logger = logging.getLogger("torchtitan_amd")

_RECIPES = {"mxfp8_rceil": "rceil", "mxfp8_floor": "floor"}


def _arch_has_capability(arch: str, major: int, minor: int) -> bool:
    """Whether the architecture string `arch` ("gfx950", "gfx950:sramecc+:xnack-") names a GPU of
    the family gfx<major><minor>x.  The family must match exactly: the kernels are written for
    one instruction set, and a larger number (gfx11xx, gfx12xx) is a different one, not a newer
    member of it."""
    digits = arch.split(":")[0].removeprefix("gfx")
    try:
        got = (int(digits[:-2]), int(digits[-2], 16))
    except (ValueError, IndexError):
        return False
    return got == (major, minor)


def has_rocm_capability(major: int, minor: int) -> bool:
    """True when the current device is an AMD GPU of the family gfx<major><minor>x
    (9, 5 -> gfx950 = MI350X / MI355X).  Stands where the reference asks
    `has_cuda_capability(10, 0)` (torchtitan/tools/utils.py:28-33)."""
    if not torch.cuda.is_available() or torch.version.hip is None:
        return False
    arch = torch.cuda.get_device_properties(torch.cuda.current_device()).gcnArchName
    return _arch_has_capability(arch, major, minor)


def _plain_state_dict_entries(module, state_dict, prefix, local_metadata):
    for name, _ in module.named_parameters(recurse=False):
        v = state_dict.get(prefix + name)
        if isinstance(v, MXFP8TrainingWeight):
            state_dict[prefix + name] = v.as_subclass(torch.Tensor)


class MXFP8Converter(QuantizationConverter):
    """Wraps the weights of target ``nn.Linear`` modules and 3-D ``nn.Parameter`` experts in a
    tensor subclass that overrides ``F.linear`` and ``torch._grouped_mm`` with dynamically
    quantized MXFP8 GEMMs."""

    @dataclass(kw_only=True, slots=True)
    class Config(QuantizationConverter.Config):
        _quantization_type: ClassVar[str] = "mxfp8"

        recipe_name: Literal["mxfp8_rceil", "mxfp8_floor"] = "mxfp8_rceil"
        """mxfp8_rceil: E8M0 scale = ceil(log2(amax / 448)) (the reference's recipe);
        mxfp8_floor: scale = floor(log2 amax) - 8 (OCP MX v1.0 default, codes may saturate)."""

        fqns: list[str] = field(default_factory=list)
        """Modules whose fully qualified name contains any of these strings are converted.
        The default (empty) converts nothing."""

        filter_fqns: list[str] = field(default_factory=list)
        """Modules whose fully qualified name contains any of these strings are left in high
        precision even when `fqns` selects them (the exclusion list the reference's low-precision
        converters carry, torchtitan/components/quantization/float8.py:51-56).  nn.Linear modules
        with a weight dimension that is not a multiple of 16 are always skipped.
        Example: fqns=["layers"], filter_fqns=["attention.wk", "attention.wv"]."""

        pad_token_groups_for_grouped_mm: bool = True
        """Pad token groups to multiples of 32 inside the grouped GEMM.  Set to false when the
        dispatcher already delivers 32-aligned groups."""

        fuse_swiglu_cast: bool = True
        """Not in the reference's Config.  A SwiGLU block whose w2 is converted forms
        silu(w1 x) * w3 x inside the cast kernel that feeds w2 (one pass over the two
        projections instead of three elementwise passes and a cast).  The bf16 gate value can
        differ from the unfused ops' by one rounding step at a few elements in ten thousand;
        false keeps the three separate ops."""

        cache_weight_casts: bool = False
        """Not in the reference's Config.  Keep the MXFP8 forms of a converted weight until the
        weight is next updated in place (2 extra bytes per weight element): `post_optimizer_hook`
        then casts every converted weight once per optimizer step, and every forward until the
        next step (gradient accumulation, evaluation, several micro-batches) and
        `export_mxfp8_state_dict` reuse those codes."""

        fuse_rmsnorm_cast: bool = False
        """Not in the reference's Config.  Lets blocks that call `mx_norm_linears` /
        `mx_norm_feed_forward` run the RMSNorm in front of converted linears inside the cast
        kernel.  Off by default because the result is not bit-identical to a separate norm (the
        float32 row reduction differs from torch's in its last bits)."""

    def __init__(self, config: Config, *, parallel_dims: Any, model_compile_enabled: bool):
        self.enabled = False
        if not _lib.LIB_PATH.exists():
            raise ImportError(
                f"{_lib.LIB_PATH.name} is not built. Run `python -m torchtitan_amd._build` "
                "to use MXFP8 linear layers."
            )
        assert has_rocm_capability(9, 5), "MXFP8 is only supported on gfx950 (MI350X/MI355X) GPUs"
        if config.recipe_name not in _RECIPES:
            raise ValueError(f"unknown recipe {config.recipe_name!r}; options: {sorted(_RECIPES)}")
        if model_compile_enabled:
            logger.info("under torch.compile a converted linear is one opaque operator per pass; cast sharing "
                        "between sibling linears and the gate / norm fusions are features of the eager path")
        self.config = config
        # which nn.Linear modules may be converted: dims % 16 and not excluded by name
        # (built as in torchtitan/components/quantization/float8.py:176)
        self.filter_fn = partial(module_filter_fn, filter_fqns=config.filter_fqns)
        self.enabled = True
        logger.info("MXFP8 training enabled")

    def _matches(self, fqn: str) -> bool:
        if any(part in fqn for part in self.config.filter_fqns):
            return False
        return any(target in fqn for target in self.config.fqns)

    def convert(self, model: nn.Module):
        """Replace, in place, the weight of every matching ``nn.Linear`` and every matching
        module's 3-D parameters by an ``MXFP8TrainingWeight`` sharing the same storage."""
        if not self.enabled:
            return
        verify_module_protocol(model, nn.Linear, Linear)
        saved = capture_module_attrs(model, ["_init_mean", "_init_std"], nn_module_cls=nn.Linear)
        cfg = MXFP8Config(_RECIPES[self.config.recipe_name],
                          self.config.pad_token_groups_for_grouped_mm,
                          self.config.fuse_swiglu_cast, self.config.cache_weight_casts,
                          self.config.fuse_rmsnorm_cast)
        n_linear = n_grouped = 0
        for fqn, mod in model.named_modules():
            if not self._matches(fqn):
                continue
            before = n_linear + n_grouped
            if isinstance(mod, nn.Linear):
                if not self.filter_fn(mod, fqn):
                    logger.warning("skipping %s: weight %s has a dimension that is not a multiple of 16",
                                   fqn, tuple(mod.weight.shape))
                    continue
                if mod.in_features % 32:
                    logger.warning("skipping %s: in_features %d is not a multiple of 32", fqn, mod.in_features)
                    continue
                mod.weight = wrap_parameter(mod.weight, cfg)
                n_linear += 1
            else:
                for name, p in list(mod.named_parameters(recurse=False)):
                    if p.dim() == 3 and not isinstance(p, MXFP8TrainingWeight):
                        setattr(mod, name, wrap_parameter(p, cfg))
                        n_grouped += 1
            if n_linear + n_grouped > before and not getattr(mod, "_mx_plain_state_dict", False):
                # checkpoints hold plain tensors: loadable without this package, also weights-only
                mod.register_state_dict_post_hook(_plain_state_dict_entries)
                mod._mx_plain_state_dict = True
        inject_module_protocol(model, Linear, saved)
        verify_module_protocol(model, nn.Linear, Linear)
        logger.info(
            "Converted %d linear weights and %d grouped expert weights matching FQNs %s "
            "to dynamic %s quantization for grouped_mm and linear ops",
            n_linear, n_grouped, self.config.fqns, self.config.recipe_name,
        )

    def post_optimizer_hook(self, model: nn.Module | list[nn.Module]):
        """Nothing to do by default: weights are re-quantized in every forward, as in the
        reference.  With `cache_weight_casts` the freshly updated weights are cast here, once per
        optimizer step, for the forwards that follow and for a hand-over in MXFP8 form."""
        if not self.enabled or not self.config.cache_weight_casts:
            return
        for m in model if isinstance(model, (list, tuple)) else [model]:
            for p in m.parameters():
                if isinstance(p, MXFP8TrainingWeight) and p.is_cuda:
                    with torch.no_grad():
                        _cast_weight(p.as_subclass(torch.Tensor), p.mx_config.scale_mode, True, p.mx_config)


MXFP8_PAYLOAD_FORMAT = "mxfp8:e4m3fn+e8m0:block32:dim-1"


def export_mxfp8_state_dict(model: nn.Module) -> dict:
    """The model's state dict with every converted weight in MXFP8 form: for such a key the
    value is ``{"format", "codes" (uint8, the weight's shape), "scales" (uint8, one E8M0 byte
    per 32 elements of the last dim, row-major), "dtype" (of the original)}`` -- 1.03 bytes per
    element instead of 2 -- and every other tensor is passed through.  What a trainer can hand
    to a generator in place of the bf16 state dict
    (torchtitan/experiments/rl/unified/actors/trainer.py:226-239)."""
    from .. import ops

    converted = {name: p for name, p in model.named_parameters() if isinstance(p, MXFP8TrainingWeight)}
    out = {}
    for name, t in model.state_dict().items():
        p = converted.get(name)
        if p is None or not p.is_cuda or p.shape[-1] % 32:
            out[name] = t
            continue
        with torch.no_grad():
            rows, _ = _cast_weight(p.as_subclass(torch.Tensor), p.mx_config.scale_mode, False, p.mx_config)
        lead = p.shape[:-1]
        n_rows, nblk = int(torch.Size(lead).numel()), p.shape[-1] // 32
        if p.dim() == 3 and p.shape[1] % 128:  # per-matrix scale blocks: undo them one by one
            per = ops.mfma_scale_bytes(p.shape[1], nblk)
            scales = torch.stack([ops.scale_unlayout(rows.scales[g * per:(g + 1) * per], p.shape[1], nblk)
                                  for g in range(p.shape[0])])
        else:
            scales = ops.scale_unlayout(rows.scales, n_rows, nblk)
        out[name] = {"format": MXFP8_PAYLOAD_FORMAT, "codes": rows.codes.view(*p.shape),
                     "scales": scales.view(*lead, nblk), "dtype": p.dtype}
    return out


def load_mxfp8_state_dict(payload: dict) -> dict:
    """Plain state dict from `export_mxfp8_state_dict`'s output: MXFP8 entries are dequantized to
    their original dtype (what `load_weights_from_state_dict` on the receiving side expects,
    torchtitan/experiments/rl/unified/actors/generator.py:307-335)."""
    from .. import ops
    from ..ops import MX_SCALES_ROWMAJOR, MXData

    out = {}
    for name, v in payload.items():
        if not (isinstance(v, dict) and v.get("format") == MXFP8_PAYLOAD_FORMAT):
            out[name] = v
            continue
        codes, scales = v["codes"], v["scales"]
        flat = ops.mx_dequant(MXData(codes.reshape(-1, codes.shape[-1]),
                                     scales.reshape(-1, scales.shape[-1]).contiguous(), MX_SCALES_ROWMAJOR))
        out[name] = flat.view(codes.shape).to(v["dtype"])
    return out
