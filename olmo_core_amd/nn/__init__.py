from .feed_forward import FeedForward, swiglu
from .moe import DroplessMoEMLP, ParallelDroplessMLP, float8_dropless_mlp

__all__ = ["FeedForward", "swiglu", "DroplessMoEMLP", "ParallelDroplessMLP", "float8_dropless_mlp"]
