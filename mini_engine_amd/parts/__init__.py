"""Model parts. Importing this package registers the built-in parts."""
from .base import (PAGE, CacheNeed, CacheView, FeedForward, Head, LayerCall, Mixer, Norm, PageTensor, ParamSpec, Part,  # noqa: F401
                   PendingNorm, PositionEncoding, StateNeed, make_part, register_part, registered)
from . import attention, block, embedding, feed_forward, linear, norms, rotary  # noqa: F401
