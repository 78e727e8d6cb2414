"""Parts a decoder is assembled from; importing the package registers the built-in kinds."""
from .base import (  # noqa: F401
    PAGE, Block, CompositeNeed, Embedding, FeedForward, Mixer, Norm, OutputHead, PagedNeed, Param, Part, PartSpec, PositionEncoding, ScaledSum, StateNeed, StreamUpdate,
    fused_rows, make_part, register_arrangement, register_part, single,
)
from . import attention, conv_attention, feed_forward, latent_attention, linear_recurrence, normed_attention, norms, parallel_mixer, position  # noqa: F401  (register kinds)
from .attention import kv_pages  # noqa: F401
from .block import HyperConnectionBlock, OutputNormBlock, ParallelBlock, PreNormBlock  # noqa: F401
from .model import DecoderModel, LayerSpec, ModelSpec, ScheduleEntry  # noqa: F401
