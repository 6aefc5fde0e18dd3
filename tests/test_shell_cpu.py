"""Host-side plugin shell: config rules, module protocol utilities, converter container and
the weight wrapper's dispatch.  These mirror what the reference's unit tests pin for the shell
(tests/unit_tests/test_linear.py:138-316, test_model_converter.py:29-68, test_configurable.py)."""
from dataclasses import dataclass, field

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import torchtitan_amd.mx_tensor as mt
from torchtitan_amd.config import Configurable
from torchtitan_amd.modules import FeedForward, GroupedExperts, Linear, compute_ffn_hidden_dim
from torchtitan_amd.modules import moe as moe_mod
from torchtitan_amd.mx_tensor import MXFP8Config, MXFP8TrainingWeight, wrap_parameter
from torchtitan_amd.protocols import ModelConvertersContainer, Module
from torchtitan_amd.quantization import MXFP8_GROUP_ALIGNMENT_SIZE, QuantizationConverter
from torchtitan_amd.quantization import mx as mx_mod
from torchtitan_amd.quantization.module_utils import (
    capture_module_attrs,
    inject_module_protocol,
    verify_module_protocol,
)
from torchtitan_amd.quantization.mx import MXFP8Converter


# ------------------------------------------------------------------ Configurable
def test_config_must_be_slotted_kw_only():
    with pytest.raises(TypeError):
        class Bad(Configurable):
            @dataclass
            class Config(Configurable.Config):
                x: int = 0


def test_build_kwargs_modes():
    class Thing(Configurable):
        @dataclass(kw_only=True, slots=True)
        class Config(Configurable.Config):
            a: int = 1
            late: int = field(init=False)

        def __init__(self, config, extra=None):
            self.config, self.extra = config, extra

    cfg = Thing.Config(a=2)
    with pytest.raises(TypeError):
        cfg.build()  # init=False slot never provided
    t = cfg.build(late=5)
    assert t.config.late == 5 and t.config.a == 2 and not hasattr(cfg, "late")
    cfg.late = 7
    assert cfg.build().config.late == 7
    with pytest.raises(ValueError):
        cfg.build(late=8)  # conflicts with the pre-set value
    assert cfg.build(extra="x").extra == "x"
    with pytest.raises(TypeError):
        cfg.build(late=7, extra="x")  # mixed
    assert "late=7" in repr(cfg) and "<UNSET>" in repr(Thing.Config())
    assert Thing.Config().to_dict() == {"a": 1}


def test_linear_requires_features_and_inits():
    with pytest.raises(TypeError):
        Linear(Linear.Config())
    lin = Linear.Config(init_std=0.03).build(in_features=64, out_features=32)
    assert isinstance(lin, nn.Linear) and isinstance(lin, Module) and lin.bias is None
    lin.init_weights()
    assert 0.02 < lin.weight.std().item() < 0.04
    lin.init_weights(init_std=0.5)
    assert lin.weight.std().item() > 0.3


def test_ffn_hidden_dim_llama3_8b():
    # torchtitan/models/llama3/__init__.py:116-144 with feed_forward.py:18-31
    assert compute_ffn_hidden_dim(4096, multiple_of=1024, ffn_dim_multiplier=1.3) == 14336


# ------------------------------------------------------------------ module_utils
class FakeQuantLinear(nn.Linear):
    pass


def test_capture_and_inject_restore_attrs():
    model = nn.Module()
    model.fc = Linear.Config(init_std=0.03).build(in_features=8, out_features=4)
    model.plain = FakeQuantLinear(8, 4)  # no _init_* attrs: not captured
    saved = capture_module_attrs(model, ["_init_mean", "_init_std"])
    assert saved == {"fc": {"_init_mean": 0.0, "_init_std": 0.03}}
    model.fc = FakeQuantLinear(8, 4)  # a conversion that builds new instances loses the attrs
    inject_module_protocol(model, Linear, saved)
    assert isinstance(model.fc, Linear) and isinstance(model.fc, FakeQuantLinear)
    assert model.fc._init_std == 0.03
    assert type(model.fc).__name__ == "FakeQuantLinear_WithLinear"


def test_inject_is_idempotent_and_caches_per_class():
    model = nn.Module()
    model.a, model.b = FakeQuantLinear(8, 4), FakeQuantLinear(4, 2)
    inject_module_protocol(model, Linear)
    assert type(model.a) is type(model.b)
    cls = type(model.a)
    inject_module_protocol(model, Linear)
    assert type(model.a) is cls


def test_class_swap_keeps_instance_attrs():
    model = nn.Module()
    model.fc = Linear.Config(init_std=0.03).build(in_features=8, out_features=4)
    model.fc.__class__ = FakeQuantLinear
    assert not isinstance(model.fc, Module) and hasattr(model.fc, "_init_std")
    inject_module_protocol(model, Linear)
    assert isinstance(model.fc, Linear) and model.fc._init_std == 0.03


def test_patched_class_cannot_be_constructed():
    model = nn.Module()
    model.fc = FakeQuantLinear(8, 4)
    inject_module_protocol(model, Linear)
    with pytest.raises(RuntimeError):
        type(model.fc)(8, 4)


def test_verify_names_offenders():
    model = nn.Module()
    model.ok = Linear.Config().build(in_features=8, out_features=4)
    verify_module_protocol(model, nn.Linear, Linear)
    model.fc1 = nn.Linear(8, 4)
    with pytest.raises(RuntimeError, match="fc1"):
        verify_module_protocol(model, nn.Linear, Linear)
    model.fc1 = FakeQuantLinear(8, 4)
    inject_module_protocol(model, Linear)
    verify_module_protocol(model, nn.Linear, Linear)


# ------------------------------------------------------------------ converter container
def _converter(monkeypatch, **cfg):
    monkeypatch.setattr(mx_mod, "has_rocm_capability", lambda *a: True)
    return MXFP8Converter.Config(**cfg)


def test_container_builds_converters(monkeypatch):
    empty = ModelConvertersContainer.Config().build(parallel_dims=None, model_compile_enabled=False)
    assert isinstance(empty, ModelConvertersContainer) and empty.converters == []
    cc = _converter(monkeypatch, fqns=["ffn"])
    box = ModelConvertersContainer.Config(converters=[cc]).build(parallel_dims=None, model_compile_enabled=False)
    assert len(box.converters) == 1 and isinstance(box.converters[0], MXFP8Converter)
    assert isinstance(box.converters[0], QuantizationConverter)
    assert box.post_optimizer_hook(nn.Module()) is None


def test_mixed_quantization_types_rejected(monkeypatch):
    class OtherQuant(QuantizationConverter):
        @dataclass(kw_only=True, slots=True)
        class Config(QuantizationConverter.Config):
            _quantization_type = "float8"

        def __init__(self, config, **kw):
            pass

    cc = _converter(monkeypatch)
    with pytest.raises(AssertionError, match="different quantization types"):
        ModelConvertersContainer.Config(converters=[cc, OtherQuant.Config()]).build(
            parallel_dims=None, model_compile_enabled=False)


def test_converter_defaults_and_gate(monkeypatch):
    cfg = MXFP8Converter.Config()
    assert cfg.recipe_name == "mxfp8_rceil" and cfg.fqns == [] and cfg.pad_token_groups_for_grouped_mm
    assert MXFP8Converter.Config._quantization_type == "mxfp8" and MXFP8_GROUP_ALIGNMENT_SIZE == 32
    monkeypatch.setattr(mx_mod, "has_rocm_capability", lambda *a: False)
    with pytest.raises(AssertionError):
        cfg.build(parallel_dims=None, model_compile_enabled=False)


class TinyBlock(Module):
    def __init__(self):
        super().__init__()
        self.attn_wq = Linear.Config().build(in_features=64, out_features=64)
        cfg = FeedForward.Config(hidden_dim=128)
        self.feed_forward = cfg.build(dim=64)
        self.experts = GroupedExperts(dim=64, hidden_dim=32, num_experts=4, use_grouped_mm=True)
        self.odd = Linear.Config().build(in_features=48, out_features=16)


def test_convert_on_meta_then_materialise(monkeypatch):
    with torch.device("meta"):
        model = TinyBlock()
    conv = _converter(monkeypatch, fqns=["feed_forward", "experts", "odd"]).build(
        parallel_dims=None, model_compile_enabled=False)
    conv.convert(model)
    ff = model.feed_forward
    assert all(isinstance(m.weight, MXFP8TrainingWeight) for m in (ff.w1, ff.w2, ff.w3))
    assert not isinstance(model.attn_wq.weight, MXFP8TrainingWeight)  # fqn not selected
    assert not isinstance(model.odd.weight, MXFP8TrainingWeight)      # 48 % 32 != 0
    assert all(isinstance(getattr(model.experts, n), MXFP8TrainingWeight) for n in ("w1", "w2", "w3"))
    assert isinstance(ff.w1, Linear) and ff.w1._init_std == 0.02
    # materialise and initialise exactly as the trainer does
    model.to_empty(device="cpu")
    ff.init_weights(init_std=0.01)
    model.experts.init_weights(init_std=0.01)
    assert isinstance(ff.w2.weight, MXFP8TrainingWeight) and isinstance(ff.w2.weight, nn.Parameter)
    assert ff.w2.weight.mx_config.scale_mode == "rceil"
    assert 0.005 < ff.w2.weight.std().item() < 0.015
    assert set(dict(model.named_parameters())) >= {"feed_forward.w1.weight", "experts.w2"}
    conv.convert(model)  # idempotent
    assert isinstance(ff.w1.weight, MXFP8TrainingWeight)


def test_default_fqns_convert_nothing(monkeypatch):
    model = TinyBlock()
    _converter(monkeypatch).build(parallel_dims=None, model_compile_enabled=False).convert(model)
    assert not any(isinstance(p, MXFP8TrainingWeight) for p in model.parameters())


# ------------------------------------------------------------------ dispatch of the wrapper
def test_wrapper_routes_linear_and_grouped_mm(monkeypatch):
    seen = []
    monkeypatch.setattr(mt, "mx_linear", lambda x, w, b, cfg: seen.append(("linear", type(w), cfg.scale_mode)) or F.linear(x, w, b))
    monkeypatch.setattr(mt, "mx_grouped_mm", lambda a, b, offs, cfg: seen.append(("grouped", tuple(b.shape), cfg.pad_token_groups_for_grouped_mm)) or torch.zeros(a.shape[0], b.shape[-1]))
    lin = nn.Linear(64, 32, bias=True)
    lin.weight = wrap_parameter(lin.weight, MXFP8Config("floor"))
    y = lin(torch.randn(4, 64))
    assert seen[-1] == ("linear", torch.Tensor, "floor") and type(y) is torch.Tensor
    w = wrap_parameter(nn.Parameter(torch.randn(4, 32, 64)), MXFP8Config("rceil", False))
    offs = torch.tensor([8, 16, 24, 32], dtype=torch.int32)
    torch._grouped_mm(torch.randn(32, 64).bfloat16(), w.bfloat16().transpose(-2, -1), offs=offs)
    assert seen[-1] == ("grouped", (4, 64, 32), False)


def test_wrapper_is_a_trainable_parameter():
    lin = nn.Linear(64, 32, bias=False)
    lin.weight = wrap_parameter(lin.weight, MXFP8Config())
    assert isinstance(lin.weight, nn.Parameter) and lin.weight.requires_grad
    before = lin.weight.detach().clone()
    opt = torch.optim.AdamW(lin.parameters(), lr=1e-2)
    (lin.weight.float() ** 2).sum().backward()
    assert type(lin.weight.grad) is torch.Tensor
    opt.step()
    assert isinstance(lin.weight, MXFP8TrainingWeight) and not torch.equal(lin.weight, before)
    assert type(lin.weight.sum()) is torch.Tensor
    sd = lin.state_dict()
    lin2 = nn.Linear(64, 32, bias=False)
    lin2.load_state_dict(sd)
    assert torch.equal(lin2.weight, lin.weight.as_subclass(torch.Tensor))


def test_mx_path_fails_loudly_without_gpu():
    """No CPU fallback: the quantized path refuses CPU tensors instead of emulating."""
    lin = nn.Linear(64, 32, bias=False)
    lin.weight = wrap_parameter(lin.weight, MXFP8Config())
    with pytest.raises(Exception, match="GPU"):
        lin(torch.randn(4, 64, dtype=torch.bfloat16))


# ------------------------------------------------------------------ MoE host glue
def test_permute_indices_host_reference_example():
    t = torch.tensor([4, 2, 1, 3, 1, 2, 3, 4])
    perm, m_sizes, m_offsets = moe_mod.generate_permute_indices(t, 4, 2, 32, 8, use_cpu=True)
    assert m_sizes.tolist() == [8, 8, 8, 8] and m_offsets.tolist() == [8, 16, 24, 32]
    assert m_sizes.dtype == torch.int32 and m_offsets.dtype == torch.int32
    assert perm.tolist() == [0, 1, 2, 3, 10, -1, -1, -1, 4, 5, 11, 12, -1, -1, -1, -1,
                             6, 13, 14, 15, -1, -1, -1, -1, 7, 8, 9, 16, 17, 18, 19, -1]


def test_alignment_switch():
    assert moe_mod.get_mxfp8_pad_multiple() is None
    moe_mod.set_token_group_alignment_size_m(32)
    try:
        assert moe_mod.get_mxfp8_pad_multiple() == 32
    finally:
        moe_mod.set_token_group_alignment_size_m(8)


def test_module_filter_fn_rules():
    """Linear only, both dims % 16, no filtered substring in the FQN (quantization/utils.py:10-27)."""
    import torch.nn as nn

    from torchtitan_amd.quantization.utils import module_filter_fn

    assert module_filter_fn(nn.Linear(32, 48), "layers.0.attention.wq", [])
    assert not module_filter_fn(nn.Linear(32, 48), "layers.0.attention.wq", ["attention.wq"])
    assert not module_filter_fn(nn.Linear(30, 48), "w", [])
    assert not module_filter_fn(nn.Linear(32, 40), "w", [])
    assert not module_filter_fn(nn.Embedding(32, 48), "tok_embeddings", [])
    assert module_filter_fn(nn.Linear(16, 16), "output", ["router"])


def test_converter_applies_filter_fqns_and_the_dims_rule(monkeypatch):
    """`filter_fqns` takes a module out of the selection `fqns` makes, and an nn.Linear with a
    weight dimension that is not a multiple of 16 is never converted (the Config field and filter
    of torchtitan/components/quantization/float8.py:51-56,176 with utils.py:10-27)."""
    cfg = MXFP8Converter.Config()
    assert cfg.filter_fqns == []

    class Block(Module):
        def __init__(self):
            super().__init__()
            self.wq = Linear.Config().build(in_features=64, out_features=64)
            self.wk = Linear.Config().build(in_features=64, out_features=32)
            self.narrow = Linear.Config().build(in_features=64, out_features=40)  # 40 % 16 != 0
            self.experts = GroupedExperts(dim=64, hidden_dim=32, num_experts=4, use_grouped_mm=True)

    class Model(Module):
        def __init__(self):
            super().__init__()
            self.layers = nn.ModuleList([Block(), Block()])
            self.output = Linear.Config().build(in_features=64, out_features=96)

    with torch.device("meta"):
        model = Model()
    conv = _converter(monkeypatch, fqns=["layers", "output"], filter_fqns=["wk", "layers.1.experts", "output"]).build(
        parallel_dims=None, model_compile_enabled=False)
    conv.convert(model)
    for i, blk in enumerate(model.layers):
        assert isinstance(blk.wq.weight, MXFP8TrainingWeight)
        assert not isinstance(blk.wk.weight, MXFP8TrainingWeight)       # excluded by name
        assert not isinstance(blk.narrow.weight, MXFP8TrainingWeight)   # 40 is not a multiple of 16
        assert isinstance(blk.experts.w1, MXFP8TrainingWeight) == (i == 0)
    assert not isinstance(model.output.weight, MXFP8TrainingWeight)
    assert conv.filter_fn(model.layers[0].wq, "layers.0.wq") and not conv.filter_fn(model.output, "output")
    verify_module_protocol(model, nn.Linear, Linear)


def test_capability_gate_wants_the_gfx95_family():
    """Exactly the CDNA4 family passes: other AMD families are different instruction sets."""
    ok = mx_mod._arch_has_capability
    assert ok("gfx950", 9, 5) and ok("gfx950:sramecc+:xnack-", 9, 5)
    for other in ("gfx942", "gfx90a", "gfx1100", "gfx1201", "gfx908", "sm_100", "", "gfx"):
        assert not ok(other, 9, 5), other


def test_converted_weights_survive_deepcopy_and_checkpoint_as_plain_tensors():
    """A converted model can be deep-copied (independent storage, still converted, still
    Parameters) and its state dict holds plain tensors: torch.save / weights-only torch.load
    round-trips it, and it loads into an unconverted model (and back) -- the parameter stays an
    ordinary high-precision one for everything but its GEMMs
    (torchtitan/components/quantization/mx.py:98-134 leaves checkpointing untouched)."""
    import copy
    import io

    import torch
    import torch.nn as nn

    from torchtitan_amd.modules import FeedForward
    from torchtitan_amd.mx_tensor import MXFP8Config, MXFP8TrainingWeight, wrap_parameter
    from torchtitan_amd.quantization.mx import _plain_state_dict_entries

    ff = FeedForward.Config(hidden_dim=64).build(dim=32)
    ff.init_weights(init_std=0.02)
    cfg = MXFP8Config("floor", False)
    for lin in (ff.w1, ff.w2, ff.w3):   # what MXFP8Converter.convert does per module (it needs a GPU)
        lin.weight = wrap_parameter(lin.weight, cfg)
        lin.register_state_dict_post_hook(_plain_state_dict_entries)
    twin = copy.deepcopy(ff)
    for a, b in zip(ff.parameters(), twin.parameters()):
        assert isinstance(b, MXFP8TrainingWeight) and isinstance(b, nn.Parameter) and b.requires_grad
        assert b.mx_config == cfg and b.data_ptr() != a.data_ptr()
        assert torch.equal(a.as_subclass(torch.Tensor), b.as_subclass(torch.Tensor))
    sd = ff.state_dict()
    assert all(type(v) is torch.Tensor for v in sd.values())
    buf = io.BytesIO()
    torch.save(sd, buf)
    buf.seek(0)
    back = torch.load(buf, weights_only=True)
    plain = FeedForward.Config(hidden_dim=64).build(dim=32)
    plain.load_state_dict(back)
    with torch.no_grad():
        for p in twin.parameters():
            p.zero_()
    twin.load_state_dict(plain.state_dict())
    for a, b in zip(ff.parameters(), twin.parameters()):
        assert isinstance(b, MXFP8TrainingWeight) and torch.equal(a.as_subclass(torch.Tensor), b.as_subclass(torch.Tensor))


def test_optimizer_state_of_converted_weights_is_plain_and_pickling_keeps_parameters():
    """AdamW's moments are made with zeros_like: they must be plain tensors, so that an optimizer
    state dict round-trips through a weights-only load; and a pickled converted Parameter comes
    back as a converted Parameter."""
    import io
    import pickle

    import torch
    import torch.nn as nn

    from torchtitan_amd.mx_tensor import MXFP8Config, MXFP8TrainingWeight, wrap_parameter

    lin = nn.Linear(32, 16, bias=False)
    lin.weight = wrap_parameter(lin.weight, MXFP8Config("floor", False))
    opt = torch.optim.AdamW(lin.parameters(), lr=1e-2)
    lin.weight.grad = torch.ones(16, 32)
    opt.step()
    state = opt.state_dict()
    moments = [v for st in state["state"].values() for v in st.values() if isinstance(v, torch.Tensor)]
    assert moments and all(type(v) is torch.Tensor for v in moments)
    buf = io.BytesIO()
    torch.save(state, buf)
    buf.seek(0)
    back = torch.load(buf, weights_only=True)
    assert torch.equal(back["state"][0]["exp_avg"], state["state"][0]["exp_avg"])
    assert isinstance(lin.weight, MXFP8TrainingWeight) and isinstance(lin.weight, nn.Parameter)
    q = pickle.loads(pickle.dumps(lin.weight))
    assert isinstance(q, nn.Parameter) and isinstance(q, MXFP8TrainingWeight) and q.requires_grad
    assert q.mx_config.scale_mode == "floor" and torch.equal(q.detach().as_subclass(torch.Tensor),
                                                              lin.weight.detach().as_subclass(torch.Tensor))
