"""
Float8 training configuration and model conversion - the ``olmo_core.float8`` surface on native kernels.

Same names and semantics as the reference module (reference: src/olmo_core/float8/__init__.py:17
``__all__``; :22-62 ``Float8Config``; :64-162 ``apply_float8_linear``): a config selects either explicit
options (``ao``), a named recipe (``ao_recipe``) or an MX config (``ao_mx``, configuration surface only
here), and ``apply_float8_linear`` swaps every eligible ``nn.Linear`` of a model in place.
"""

from __future__ import annotations

import logging
from dataclasses import dataclass
from typing import List, Optional, Set

import torch.nn as nn

from ..config import Config
from ..exceptions import OLMoConfigurationError
from .ao import AOFloat8LinearConfig, AOFloat8LinearRecipe, AOMXLinearConfig

__all__ = [
    "Float8Config",
    "AOFloat8LinearConfig",
    "AOFloat8LinearRecipe",
    "AOMXLinearConfig",
    "precompute_float8_dynamic_scale_for_fsdp",
]


def precompute_float8_dynamic_scale_for_fsdp(module: nn.Module) -> None:
    """See :func:`olmo_core_amd.float8.linear.precompute_float8_dynamic_scale_for_fsdp`."""
    from .linear import precompute_float8_dynamic_scale_for_fsdp as impl

    impl(module)

log = logging.getLogger(__name__)


@dataclass
class Float8Config(Config):
    """
    Float8 options.

    :param ao: explicit float8 linear options.
    :param ao_recipe: alternatively, a named recipe.
    :param ao_mx: MX-format options (accepted as configuration; applying them raises, there is no
        native MX path).
    :param modules_to_ignore: fully-qualified names of Linear modules to leave in high precision.
    :param enabled: if ``False`` applying the config is a no-op.
    """

    ao: Optional[AOFloat8LinearConfig] = None
    ao_recipe: Optional[AOFloat8LinearRecipe] = None
    ao_mx: Optional[AOMXLinearConfig] = None
    modules_to_ignore: Optional[List[str]] = None
    enabled: bool = True

    def __post_init__(self):
        self.validate()

    def validate(self):
        chosen = [c for c in (self.ao, self.ao_recipe, self.ao_mx) if c is not None]
        if len(chosen) > 1:
            raise OLMoConfigurationError("'ao', 'ao_recipe', and 'ao_mx' configs are mutually exclusive")

    @property
    def should_precompute_float8_dynamic_scale_for_fsdp(self) -> bool:
        if self.ao_recipe is not None or self.ao_mx is not None:
            return False
        resolved = (self.ao if self.ao is not None else AOFloat8LinearConfig()).to_ao_type()
        return resolved.enable_fsdp_float8_all_gather

    def _resolve(self):
        from .native_config import Float8LinearConfig

        if self.ao_recipe is not None:
            return Float8LinearConfig.from_recipe_name(self.ao_recipe.to_ao_type())
        return (self.ao if self.ao is not None else AOFloat8LinearConfig()).to_ao_type()

    def apply_float8_linear(self, model: nn.Module, *, modules_to_ignore: Optional[Set[str]] = None):
        """
        Convert the linear layers of ``model`` to :class:`~olmo_core_amd.float8.linear.Float8Linear`,
        mutating the model in place.  Call it before compiling, activation checkpointing or wrapping the
        model in any parallel wrapper.  A Linear is left alone if its name is in ``modules_to_ignore`` or
        if any dimension of its weight is not a multiple of 16; names in ``modules_to_ignore`` that match
        no Linear are an error.  Parameters frozen before the call stay frozen.
        """
        if not self.enabled:
            return

        self.validate()
        if self.ao_mx is not None:
            raise RuntimeError("MX format training has no native gfx950 path in this library")

        from .linear import convert_to_float8_training

        seen_ignored: Set[str] = set()

        def keep_or_convert(m: nn.Module, fqn: str) -> bool:
            if modules_to_ignore is not None and fqn in modules_to_ignore:
                seen_ignored.add(fqn)
                return False
            if isinstance(m, nn.Linear) and any(d % 16 != 0 for d in m.weight.shape):
                return False
            return True

        frozen = [n for n, p in model.named_parameters() if not p.requires_grad]

        convert_to_float8_training(model, config=self._resolve(), module_filter_fn=keep_or_convert)

        if modules_to_ignore is not None and modules_to_ignore != seen_ignored:
            raise OLMoConfigurationError(
                f"invalid module name(s) in 'modules_to_ignore': {list(modules_to_ignore - seen_ignored)}"
            )
        if seen_ignored:
            log.info(f"Ignored modules for Float8 conversion: {sorted(seen_ignored)}")
        for n in frozen:
            model.get_parameter(n).requires_grad = False
