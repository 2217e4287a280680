"""Configuration boundary: Config base semantics (reference: src/test/config_test.py:7-101), AO mirror
translation (reference: src/test/float8/ao_test.py:14-48) and the model swap / filter rules
(reference: src/olmo_core/float8/__init__.py:86-98, 152-162)."""

from dataclasses import dataclass
from typing import List, Optional, Set, Tuple

import pytest
import torch
import torch.nn as nn

from olmo_core_amd.config import Config, DType
from olmo_core_amd.exceptions import OLMoConfigurationError
from olmo_core_amd.float8 import AOFloat8LinearConfig, AOFloat8LinearRecipe, AOMXLinearConfig, Float8Config
from olmo_core_amd.float8.ao import (
    AOCastConfig,
    AOFloat8GemmConfig,
    AOMXFP8Dim1CastKernelChoice,
    AOScaleCalculationMode,
    AOScalingGranularity,
    AOScalingType,
)
from olmo_core_amd.float8.linear import Float8Linear, convert_to_float8_training
from olmo_core_amd.float8.native_config import (
    Float8LinearConfig,
    ScalingGranularity,
    ScalingType,
)
from oracle import float8_oracle as O


@dataclass
class Bar:
    x: int
    y: int
    _z: int = 0


@dataclass
class Foo(Config):
    bar: Bar
    z: str


@dataclass
class CBar(Config):
    x: int
    y: int


@dataclass
class CFoo(Config):
    bar: CBar
    z: str


def test_simple_config_as_dict():
    @dataclass
    class MockConfig(Config):
        name: str = "default"
        x: Optional[int] = None

    c = MockConfig()
    assert c.as_dict() == dict(name="default", x=None)
    assert c.as_dict(exclude_none=True) == dict(name="default")


def test_nested_configs():
    foo = Foo(bar=Bar(x=1, y=2), z="z")
    data = foo.as_dict()
    assert isinstance(data["bar"], dict)
    foo1 = Foo.from_dict(data)
    assert foo1 == foo and isinstance(foo1.bar, Bar)
    foo2 = Foo.from_dict(data, overrides=["bar.x=0"])
    assert foo2.bar.x == 0
    assert foo2.merge(["bar.x=-1"]).bar.x == -1
    assert foo.as_dict(recurse=False) == {"z": "z", "bar": foo.bar}
    assert foo.as_config_dict() == {
        Config.CLASS_NAME_FIELD: f"{__name__}.Foo",
        "z": "z",
        "bar": {Config.CLASS_NAME_FIELD: f"{__name__}.Bar", "x": 1, "y": 2},
    }


def test_json_safe_dump():
    @dataclass
    class Coll(Config):
        x_list: List[int]
        x_tuple: Tuple[int, ...]
        x_set: Set[str]

    c = Coll(x_list=[0, 1], x_tuple=(0, 1), x_set={"a"})
    d = c.as_config_dict()
    d.pop(Config.CLASS_NAME_FIELD)
    assert d == {"x_list": [0, 1], "x_tuple": [0, 1], "x_set": ["a"]}


def test_non_strict_merge_and_prefix():
    foo = CFoo(bar=CBar(x=1, y=2), z="a").merge(["--z=b", "--bar.x=0", "--baz.booz=0"], strict=False)
    assert foo.z == "b" and foo.bar.x == 0
    foo = CFoo(bar=CBar(x=1, y=2), z="a").merge(["--foo.z=b", "--foo.bar.x=0"], prefix="foo")
    assert foo.z == "b" and foo.bar.x == 0


def test_dtype_enum():
    assert DType.float8_e4m3fn.as_pt() == torch.float8_e4m3fn
    assert DType.from_pt(torch.float8_e5m2) == DType.float8_e5m2
    assert str(DType.bfloat16) == "bfloat16"


# ---- AO mirrors ------------------------------------------------------------------------------------


def test_ao_float8_linear_config_translation():
    assert isinstance(AOFloat8LinearConfig().to_ao_type(), Float8LinearConfig)
    assert AOFloat8LinearConfig(emulate=True).to_ao_type().emulate
    resolved = AOFloat8LinearConfig(cast_config_input=AOCastConfig(scaling_type=AOScalingType.disabled)).to_ao_type()
    assert resolved.cast_config_input.scaling_type == ScalingType.DISABLED
    rec = AOFloat8LinearConfig.recommended()
    assert rec.enable_fsdp_float8_all_gather and rec.force_recompute_fp8_weight_in_bwd and rec.round_scales_to_power_of_2
    r = rec.to_ao_type()
    assert r.enable_fsdp_float8_all_gather and r.round_scales_to_power_of_2


def test_ao_defaults_and_dtypes():
    c = AOFloat8LinearConfig().to_ao_type()
    assert c.cast_config_input.target_dtype == torch.float8_e4m3fn
    assert c.cast_config_weight.target_dtype == torch.float8_e4m3fn
    assert c.cast_config_grad_output.target_dtype == torch.float8_e5m2
    assert c.cast_config_grad_output_for_grad_weight.target_dtype == torch.float8_e5m2
    assert not c.round_scales_to_power_of_2 and not c.emulate and not c.enable_fsdp_float8_all_gather
    assert AOFloat8GemmConfig().to_ao_type().use_fast_accum is False
    c = AOFloat8LinearConfig(
        cast_config_grad_output=AOCastConfig(target_dtype=DType.float8_e4m3fn,
                                             scaling_granularity=AOScalingGranularity.axiswise)
    ).to_ao_type()
    assert c.cast_config_grad_output.target_dtype == torch.float8_e4m3fn
    assert c.cast_config_grad_output.scaling_granularity == ScalingGranularity.AXISWISE
    assert c.cast_config_grad_output_for_grad_weight.scaling_granularity == ScalingGranularity.AXISWISE


@pytest.mark.parametrize("name", ["tensorwise", "rowwise", "rowwise_with_gw_hp"])
def test_recipes_match_oracle_restatement(name):
    ours = Float8LinearConfig.from_recipe_name(AOFloat8LinearRecipe(name).to_ao_type())
    ref = O.recipe(name)
    pairs = [
        (ours.cast_config_input, ref.input), (ours.cast_config_weight, ref.weight),
        (ours.cast_config_grad_output, ref.grad_output),
        (ours.cast_config_input_for_grad_weight, ref.input_for_grad_weight),
        (ours.cast_config_weight_for_grad_input, ref.weight_for_grad_input),
        (ours.cast_config_grad_output_for_grad_weight, ref.grad_output_for_grad_weight),
    ]
    for a, b in pairs:
        assert a.scaling_type.value == b.scaling_type
        assert a.scaling_granularity.value == b.granularity
        if b.scaling_type != O.DISABLED:
            assert a.target_dtype == b.dtype
    assert ours.round_scales_to_power_of_2 == ref.round_scales_to_power_of_2


def test_invalid_configs():
    with pytest.raises(ValueError, match="incompatible operand precision"):
        bad = AOFloat8LinearConfig(cast_config_input=AOCastConfig(scaling_type=AOScalingType.disabled))
        Float8Config(ao=bad).apply_float8_linear(nn.Linear(16, 16))
    with pytest.raises(ValueError):
        AOFloat8LinearConfig(
            enable_fsdp_float8_all_gather=True,
            cast_config_weight=AOCastConfig(scaling_granularity=AOScalingGranularity.axiswise),
        ).to_ao_type()
    with pytest.raises(OLMoConfigurationError):
        Float8Config(ao=AOFloat8LinearConfig(), ao_recipe=AOFloat8LinearRecipe.rowwise)


def test_mx_config_surface_only():
    mx = AOMXLinearConfig.mxfp8_cublas_rceil()
    assert mx.mxfp8_cast_kernel_choice == AOMXFP8Dim1CastKernelChoice.cuda
    assert mx.scale_calculation_mode == AOScaleCalculationMode.rceil
    with pytest.raises(NotImplementedError):
        AOMXLinearConfig(block_size=32).to_ao_type()
    with pytest.raises(RuntimeError):
        Float8Config(ao_mx=mx).apply_float8_linear(nn.Linear(16, 16))


def test_float8_config_roundtrip_and_flags():
    cfg = Float8Config(ao=AOFloat8LinearConfig.recommended(), modules_to_ignore=["a.b"])
    again = Float8Config.from_dict(cfg.as_config_dict())
    assert again == cfg
    assert cfg.should_precompute_float8_dynamic_scale_for_fsdp
    assert not Float8Config().should_precompute_float8_dynamic_scale_for_fsdp
    assert not Float8Config(ao_recipe=AOFloat8LinearRecipe.tensorwise).should_precompute_float8_dynamic_scale_for_fsdp
    merged = Float8Config().merge(["--enabled=false"])
    assert merged.enabled is False


# ---- swap / filter ---------------------------------------------------------------------------------


class Toy(nn.Module):
    def __init__(self):
        super().__init__()
        self.blocks = nn.ModuleList([nn.ModuleDict({"w1": nn.Linear(32, 64), "w2": nn.Linear(64, 32)}) for _ in range(2)])
        self.odd = nn.Linear(32, 10)       # 10 is not a multiple of 16
        self.lm_head = nn.Linear(32, 48)
        self.norm = nn.LayerNorm(32)


def _converted(m):
    return sorted(n for n, mod in m.named_modules() if isinstance(mod, Float8Linear))


def test_apply_float8_linear_swaps_expected_modules():
    m = Toy()
    w_before = m.blocks[0]["w1"].weight
    Float8Config().apply_float8_linear(m, modules_to_ignore={"lm_head"})
    assert _converted(m) == sorted(O.expected_swaps(Toy(), ["lm_head"]))
    assert _converted(m) == ["blocks.0.w1", "blocks.0.w2", "blocks.1.w1", "blocks.1.w2"]
    assert m.blocks[0]["w1"].weight is w_before
    assert isinstance(m.odd, nn.Linear) and not isinstance(m.odd, Float8Linear)
    assert set(m.state_dict().keys()) == set(Toy().state_dict().keys())


def test_apply_float8_linear_disabled_is_noop():
    m = Toy()
    Float8Config(enabled=False).apply_float8_linear(m)
    assert _converted(m) == []


def test_invalid_ignore_name_raises():
    with pytest.raises(OLMoConfigurationError, match="invalid module name"):
        Float8Config().apply_float8_linear(Toy(), modules_to_ignore={"lm_head", "nope"})


def test_frozen_params_stay_frozen_and_meta_device_works():
    with torch.device("meta"):
        m = Toy()
    m.blocks[0]["w1"].weight.requires_grad_(False)
    Float8Config(ao=AOFloat8LinearConfig.recommended()).apply_float8_linear(m, modules_to_ignore=set())
    assert m.blocks[0]["w1"].weight.requires_grad is False
    assert m.blocks[0]["w1"].weight.is_meta and isinstance(m.blocks[0]["w1"], Float8Linear)


def test_root_linear_and_filter_sees_only_linears():
    seen = []

    def filt(mod, fqn):
        seen.append((type(mod).__name__, fqn))
        return True

    root = convert_to_float8_training(nn.Linear(16, 16), module_filter_fn=filt)
    assert isinstance(root, Float8Linear) and seen == [("Linear", "")]
    seen.clear()
    convert_to_float8_training(Toy(), module_filter_fn=filt)
    assert all(kind == "Linear" for kind, _ in seen)
    assert [n for _, n in seen] == ["blocks.0.w1", "blocks.0.w2", "blocks.1.w1", "blocks.1.w2", "odd", "lm_head"]


def test_emulate_is_refused_at_conversion():
    with pytest.raises(NotImplementedError):
        Float8Config(ao=AOFloat8LinearConfig(emulate=True)).apply_float8_linear(Toy())


def test_no_cpu_path():
    m = Toy()
    Float8Config().apply_float8_linear(m, modules_to_ignore={"lm_head"})
    with pytest.raises(RuntimeError, match="no CPU path"):
        m.blocks[0]["w1"](torch.randn(4, 32))


def test_kept_weight_operands_need_the_switch_and_a_gpu_weight():
    """Float8Linear.weight_operands(): nothing is kept without enable_fsdp_float8_all_gather, and a weight that
    is not on the GPU is never quantised ahead of the forward (which then raises: there is no CPU path)."""
    import torch.nn as nn

    from olmo_core_amd.float8 import AOFloat8LinearConfig, Float8Config
    from olmo_core_amd.float8.linear import Float8Linear

    for cfg in (AOFloat8LinearConfig(), AOFloat8LinearConfig.recommended()):
        model = nn.Sequential(nn.Linear(32, 48, bias=False))
        Float8Config(ao=cfg).apply_float8_linear(model)
        assert isinstance(model[0], Float8Linear)
        assert model[0].weight_operands() is None


def test_product_never_reaches_for_the_checker_or_working_files():
    """The package (Python and HIP sources) imports, reads and names nothing under oracle/ or _work/: the oracle is
    test infrastructure, working files are not part of the repository."""
    import re
    from pathlib import Path

    pkg = Path(__file__).resolve().parent.parent / "olmo_core_amd"
    offenders = []
    for path in pkg.rglob("*"):
        if path.suffix not in (".py", ".hip", ".h") or "__pycache__" in path.parts:
            continue
        text = path.read_text()
        if re.search(r"\b(from|import)\s+oracle\b|oracle/|_work/|liboracle", text):
            offenders.append(str(path.relative_to(pkg)))
    assert offenders == []
