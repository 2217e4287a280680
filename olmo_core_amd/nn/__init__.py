from .feed_forward import FeedForward, swiglu

__all__ = ["FeedForward", "swiglu"]
