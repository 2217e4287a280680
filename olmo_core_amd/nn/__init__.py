from .feed_forward import FeedForward, swiglu
from .moe import DroplessMoEMLP, float8_dropless_mlp

__all__ = ["FeedForward", "swiglu", "DroplessMoEMLP", "float8_dropless_mlp"]
