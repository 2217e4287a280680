"""
olmo_core_amd - MI355X-native float8 linear path behind the ``olmo_core.float8`` interface.

    from olmo_core_amd.float8 import Float8Config, AOFloat8LinearConfig, AOFloat8LinearRecipe
    Float8Config(ao_recipe=AOFloat8LinearRecipe.tensorwise).apply_float8_linear(model)

All arithmetic runs in hand-written gfx950 HIP kernels behind the C ABI of ``libmi8.so``
(``include/mi8.h``); there is no CPU or eager-PyTorch fallback.
"""

from .exceptions import MI8KernelError, OLMoConfigurationError

__all__ = ["MI8KernelError", "OLMoConfigurationError", "__version__"]
__version__ = "0.1.0"
