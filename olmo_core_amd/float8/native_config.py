"""
Resolved configuration of the native float8 linear path.

These are the objects the ``AO*`` mirror dataclasses translate into (``to_ao_type()``); they play the
role that torchao's ``torchao.float8.config`` types play for the reference
(reference: src/olmo_core/float8/ao.py:27-51 translation, :54-109 enums, :152-186 the 14 fields).
Field names, defaults and the recipe table follow torchao 0.15.0's ``Float8LinearConfig``:
everything dynamic + tensorwise, e4m3 for input and weight, e5m2 for grad_output, the
``*_for_grad_*`` casts default to their base cast, ``emulate`` / ``pad_inner_dim`` /
``enable_fsdp_float8_all_gather`` / ``round_scales_to_power_of_2`` off.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass, replace
from typing import Optional

import torch

__all__ = [
    "ScalingType",
    "ScalingGranularity",
    "CastConfig",
    "Float8GemmConfig",
    "Float8LinearRecipeName",
    "Float8LinearConfig",
    "e4m3_dtype",
    "e5m2_dtype",
]

# gfx950 implements the OCP encodings natively (the fnuz variants belong to gfx942).
e4m3_dtype = torch.float8_e4m3fn
e5m2_dtype = torch.float8_e5m2


class ScalingType(enum.Enum):
    DYNAMIC = "dynamic"
    DISABLED = "disabled"

    def short_str(self) -> str:
        return "dyn" if self is ScalingType.DYNAMIC else "dis"


class ScalingGranularity(enum.Enum):
    TENSORWISE = "tensorwise"
    AXISWISE = "axiswise"

    def short_str(self) -> str:
        return "ten" if self is ScalingGranularity.TENSORWISE else "axs"


@dataclass
class CastConfig:
    """How one operand of one GEMM is quantised."""

    scaling_type: ScalingType = ScalingType.DYNAMIC
    scaling_granularity: ScalingGranularity = ScalingGranularity.TENSORWISE
    target_dtype: Optional[torch.dtype] = None

    def short_str(self) -> str:
        dt = {e4m3_dtype: "e4m3", e5m2_dtype: "e5m2", None: "none"}[self.target_dtype]
        return f"{self.scaling_type.short_str()}_{self.scaling_granularity.short_str()}_{dt}"

    def __post_init__(self):
        if self.scaling_granularity is ScalingGranularity.AXISWISE:
            if self.scaling_type is not ScalingType.DYNAMIC:
                raise ValueError("axiswise scaling requires dynamic scaling")
        if self.target_dtype is not None and self.target_dtype not in (e4m3_dtype, e5m2_dtype):
            raise ValueError(f"unsupported float8 dtype {self.target_dtype}")


@dataclass(frozen=True)
class Float8GemmConfig:
    """Per-GEMM options.  ``use_fast_accum`` is accepted for interface parity; the MFMA path always
    accumulates in full fp32, so it has no numerical effect here."""

    use_fast_accum: bool = False


class Float8LinearRecipeName(enum.Enum):
    TENSORWISE = "tensorwise"
    ROWWISE = "rowwise"
    ROWWISE_WITH_GW_HP = "rowwise_with_gw_hp"


@dataclass
class Float8LinearConfig:
    cast_config_input: CastConfig = None  # type: ignore[assignment]
    cast_config_input_for_grad_weight: Optional[CastConfig] = None
    cast_config_weight: CastConfig = None  # type: ignore[assignment]
    cast_config_weight_for_grad_input: Optional[CastConfig] = None
    cast_config_grad_output: CastConfig = None  # type: ignore[assignment]
    cast_config_grad_output_for_grad_weight: Optional[CastConfig] = None
    gemm_config_output: Float8GemmConfig = Float8GemmConfig(use_fast_accum=True)
    gemm_config_grad_input: Float8GemmConfig = Float8GemmConfig()
    gemm_config_grad_weight: Float8GemmConfig = Float8GemmConfig()
    enable_fsdp_float8_all_gather: bool = False
    pad_inner_dim: bool = False
    emulate: bool = False
    force_recompute_fp8_weight_in_bwd: bool = False  # deprecated upstream, no effect
    round_scales_to_power_of_2: bool = False

    def __post_init__(self):
        for name in ("cast_config_input", "cast_config_weight", "cast_config_grad_output"):
            if getattr(self, name) is None:
                setattr(self, name, CastConfig())
            else:  # never alias a caller's object: the dtype defaults below are written in place
                setattr(self, name, replace(getattr(self, name)))
        for name, base in (
            ("cast_config_input_for_grad_weight", "cast_config_input"),
            ("cast_config_weight_for_grad_input", "cast_config_weight"),
            ("cast_config_grad_output_for_grad_weight", "cast_config_grad_output"),
        ):
            cur = getattr(self, name)
            setattr(self, name, replace(getattr(self, base) if cur is None else cur))

        for name in (
            "cast_config_input",
            "cast_config_input_for_grad_weight",
            "cast_config_weight",
            "cast_config_weight_for_grad_input",
        ):
            c = getattr(self, name)
            if c.target_dtype is None:
                c.target_dtype = e4m3_dtype
        for name in ("cast_config_grad_output", "cast_config_grad_output_for_grad_weight"):
            c = getattr(self, name)
            if c.target_dtype is None:
                c.target_dtype = e5m2_dtype

        # The same tensor quantised for two GEMMs must use one dtype.
        for a, b, what in (
            (self.cast_config_input, self.cast_config_input_for_grad_weight, "input"),
            (self.cast_config_weight, self.cast_config_weight_for_grad_input, "weight"),
            (self.cast_config_grad_output, self.cast_config_grad_output_for_grad_weight, "grad_output"),
        ):
            both_on = a.scaling_type is ScalingType.DYNAMIC and b.scaling_type is ScalingType.DYNAMIC
            if both_on and a.target_dtype != b.target_dtype:
                raise ValueError(f"{what} must be cast to a single float8 dtype")

        if self.enable_fsdp_float8_all_gather:
            if self.cast_config_weight.scaling_granularity is ScalingGranularity.AXISWISE:
                raise ValueError("float8 all-gather requires tensorwise weight scaling")
    def check_gemm_operands(self) -> None:
        """Both operands of one GEMM are quantised, or neither is.  Checked when a module is converted (the
        configuration itself may be built and serialised in any state, as the reference's translation test
        expects, reference: src/test/float8/ao_test.py:20-25)."""
        pairs = (
            (self.cast_config_input, self.cast_config_weight, "output"),
            (self.cast_config_grad_output, self.cast_config_weight_for_grad_input, "grad_input"),
            (self.cast_config_grad_output_for_grad_weight, self.cast_config_input_for_grad_weight, "grad_weight"),
        )
        for a, b, gemm in pairs:
            if (a.scaling_type is ScalingType.DISABLED) != (b.scaling_type is ScalingType.DISABLED):
                raise ValueError(f"incompatible operand precision for the {gemm} gemm")

    @property
    def any_axiswise(self) -> bool:
        return any(
            c.scaling_granularity is ScalingGranularity.AXISWISE
            for c in (
                self.cast_config_input,
                self.cast_config_input_for_grad_weight,
                self.cast_config_weight,
                self.cast_config_weight_for_grad_input,
                self.cast_config_grad_output,
                self.cast_config_grad_output_for_grad_weight,
            )
        )

    @staticmethod
    def from_recipe_name(recipe_name) -> "Float8LinearConfig":
        if isinstance(recipe_name, str):
            recipe_name = Float8LinearRecipeName(recipe_name)
        if recipe_name is Float8LinearRecipeName.TENSORWISE:
            return Float8LinearConfig()
        axis = lambda: CastConfig(  # noqa: E731
            scaling_granularity=ScalingGranularity.AXISWISE, target_dtype=e4m3_dtype
        )
        if recipe_name is Float8LinearRecipeName.ROWWISE:
            return Float8LinearConfig(
                cast_config_input=axis(),
                cast_config_weight=axis(),
                cast_config_grad_output=axis(),
                gemm_config_output=Float8GemmConfig(use_fast_accum=True),
                gemm_config_grad_input=Float8GemmConfig(use_fast_accum=True),
                gemm_config_grad_weight=Float8GemmConfig(use_fast_accum=True),
                round_scales_to_power_of_2=True,
            )
        if recipe_name is Float8LinearRecipeName.ROWWISE_WITH_GW_HP:
            return Float8LinearConfig(
                cast_config_input=axis(),
                cast_config_weight=axis(),
                cast_config_grad_output=axis(),
                cast_config_weight_for_grad_input=CastConfig(scaling_granularity=ScalingGranularity.TENSORWISE),
                cast_config_input_for_grad_weight=CastConfig(scaling_type=ScalingType.DISABLED),
                cast_config_grad_output_for_grad_weight=CastConfig(scaling_type=ScalingType.DISABLED),
                round_scales_to_power_of_2=True,
            )
        raise ValueError(recipe_name)
