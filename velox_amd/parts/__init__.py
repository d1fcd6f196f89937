"""Parts a decoder is assembled from; importing the package registers the built-in kinds."""
from .base import (  # noqa: F401
    PAGE, Block, Embedding, FeedForward, Mixer, Norm, OutputHead, PagedNeed, Param, Part, PartSpec, PositionEncoding, StateNeed,
    fused_rows, make_part, register_arrangement, register_part, single,
)
from . import attention, feed_forward, norms, position  # noqa: F401  (register kinds)
from .attention import kv_pages  # noqa: F401
from .block import PreNormBlock  # noqa: F401
from .model import DecoderModel, LayerSpec, ModelSpec, ScheduleEntry  # noqa: F401
