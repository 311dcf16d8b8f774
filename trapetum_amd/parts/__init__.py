"""Parts that layers are put together from; importing this package registers the built-in ones."""
from . import attention, blocks, conv, embedding, experts, feedforward, latent_attention, matrix_memory, norms, parallel, rope, state_space, time_mix   # noqa: F401
from .base import Block, Conv, Embedding, FeedForward, Head, Mixer, Norm, Part, Position   # noqa: F401
