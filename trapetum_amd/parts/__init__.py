"""Parts that layers are put together from; importing this package registers the built-in ones."""
from . import attention, blocks, embedding, feedforward, norms, rope   # noqa: F401
from .base import Block, Embedding, FeedForward, Head, Mixer, Norm, Part, Position   # noqa: F401
