"""
Serialisable mirrors of the float8 linear configuration.

Same dataclasses, enum members, field names and defaults as the reference's mirrors of torchao's
config types (reference: src/olmo_core/float8/ao.py:54-109 enums and cast/gemm configs, :152-186
``AOFloat8LinearConfig`` and ``recommended()``, :189-239 ``AOMXLinearConfig``).  ``to_ao_type()``
resolves a mirror into the native objects of ``native_config`` instead of torchao's: unset
(``None``) fields take the native default, nested mirrors and ``DType`` values are translated
recursively (reference: src/olmo_core/float8/ao.py:27-51).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional

from ..config import Config, DType, StrEnum
from . import native_config as nc

__all__ = [
    "AOScalingType",
    "AOScalingGranularity",
    "AOCastConfig",
    "AOFloat8GemmConfig",
    "AOFloat8LinearRecipe",
    "AOFloat8LinearConfig",
    "AOKernelPreference",
    "AOMXFP8Dim1CastKernelChoice",
    "AOScaleCalculationMode",
    "AOMXLinearConfig",
]


class _NativeMirror:
    """Mixin: a config (or enum) that knows which native type it stands for."""

    @property
    def ao_type(self):
        raise NotImplementedError

    def to_ao_type(self):
        target = self.ao_type
        if isinstance(self, Config):
            kwargs: Dict[str, Any] = {}
            for name, value in self.as_dict(exclude_none=True, recurse=False).items():
                if isinstance(value, _NativeMirror):
                    value = value.to_ao_type()
                elif isinstance(value, DType):
                    value = value.as_pt()
                kwargs[name] = value
            return target(**kwargs)
        if isinstance(self, StrEnum):
            for member in target:
                if member.value == self.value:
                    return member
            raise ValueError(self)
        raise NotImplementedError(type(self))


class AOScalingType(_NativeMirror, StrEnum):
    dynamic = "dynamic"
    disabled = "disabled"

    @property
    def ao_type(self):
        return nc.ScalingType


class AOScalingGranularity(_NativeMirror, StrEnum):
    tensorwise = "tensorwise"
    axiswise = "axiswise"

    @property
    def ao_type(self):
        return nc.ScalingGranularity


@dataclass
class AOCastConfig(Config, _NativeMirror):
    scaling_type: Optional[AOScalingType] = None
    scaling_granularity: Optional[AOScalingGranularity] = None
    target_dtype: Optional[DType] = None

    @property
    def ao_type(self):
        return nc.CastConfig


@dataclass
class AOFloat8GemmConfig(Config, _NativeMirror):
    use_fast_accum: Optional[bool] = False

    @property
    def ao_type(self):
        return nc.Float8GemmConfig


class AOFloat8LinearRecipe(_NativeMirror, StrEnum):
    tensorwise = "tensorwise"
    rowwise = "rowwise"
    rowwise_with_gw_hp = "rowwise_with_gw_hp"

    @property
    def ao_type(self):
        return nc.Float8LinearRecipeName


@dataclass
class AOFloat8LinearConfig(Config, _NativeMirror):
    """The 14 options of the float8 linear path; ``None`` means "native default"."""

    cast_config_input: Optional[AOCastConfig] = None
    cast_config_input_for_grad_weight: Optional[AOCastConfig] = None
    cast_config_weight: Optional[AOCastConfig] = None
    cast_config_weight_for_grad_input: Optional[AOCastConfig] = None
    cast_config_grad_output: Optional[AOCastConfig] = None
    cast_config_grad_output_for_grad_weight: Optional[AOCastConfig] = None
    gemm_config_output: Optional[AOFloat8GemmConfig] = None
    gemm_config_grad_input: Optional[AOFloat8GemmConfig] = None
    gemm_config_grad_weight: Optional[AOFloat8GemmConfig] = None
    enable_fsdp_float8_all_gather: Optional[bool] = None
    pad_inner_dim: Optional[bool] = None
    emulate: Optional[bool] = None
    force_recompute_fp8_weight_in_bwd: Optional[bool] = None  # deprecated, no effect
    round_scales_to_power_of_2: Optional[bool] = None

    @staticmethod
    def recommended(**kwargs: Any) -> "AOFloat8LinearConfig":
        return AOFloat8LinearConfig(
            enable_fsdp_float8_all_gather=True,
            force_recompute_fp8_weight_in_bwd=True,
            round_scales_to_power_of_2=True,
            **kwargs,
        )

    @property
    def ao_type(self):
        return nc.Float8LinearConfig


# ---- MX formats: configuration surface only --------------------------------------------------
# The reference gates MX training on NVIDIA SM100 (src/olmo_core/float8/__init__.py:118-120); the
# mirrors exist so that configs naming them still load, but there is no native MX path and
# ``to_ao_type`` says so.


class _MXUnsupported(_NativeMirror):
    @property
    def ao_type(self):
        raise NotImplementedError("MX formats have no native gfx950 path in this library")


class AOKernelPreference(_MXUnsupported, StrEnum):
    emulated = "emulated"
    auto = "auto"
    cuda = "cuda"
    torch = "torch"


class AOMXFP8Dim1CastKernelChoice(_MXUnsupported, StrEnum):
    torch = "torch"
    cuda = "cuda"
    triton = "triton"


class AOScaleCalculationMode(_MXUnsupported, StrEnum):
    floor = "floor"
    rceil = "rceil"
    ceil = "ceil"
    even = "even"


@dataclass
class AOMXLinearConfig(Config, _MXUnsupported):
    block_size: Optional[int] = None
    elem_dtype: Optional[DType] = None
    elem_dtype_weight_override: Optional[DType] = None
    elem_dtype_grad_output_override: Optional[DType] = None
    kernel_preference: Optional[AOKernelPreference] = None
    mxfp8_cast_kernel_choice: Optional[AOMXFP8Dim1CastKernelChoice] = None
    scale_calculation_mode: Optional[AOScaleCalculationMode] = None

    @classmethod
    def mxfp8_cublas_rceil(cls, **kwargs: Any) -> "AOMXLinearConfig":
        return AOMXLinearConfig(
            mxfp8_cast_kernel_choice=AOMXFP8Dim1CastKernelChoice.cuda,
            scale_calculation_mode=AOScaleCalculationMode.rceil,
            **kwargs,
        )
