"""Parts a model is put together from.  Importing the package registers the
built-in parts under their names."""

from tokasaurus_amd.parts import attention, block, embedding, feedforward, norm, position  # noqa: F401
from tokasaurus_amd.parts.base import (  # noqa: F401
    BLOCKS,
    EMBEDDINGS,
    HEADS,
    FEED_FORWARDS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    CacheNeed,
    CacheView,
    Normed,
    Prepared,
    PartSpec,
    StateNeed,
    StepContext,
    TensorSpec,
)
