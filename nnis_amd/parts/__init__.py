"""Parts a decoder is put together from.  Importing the package registers the
kinds the library ships."""

from .base import (  # noqa: F401
    Block,
    FeedForward,
    KVRequest,
    Mixer,
    Norm,
    Part,
    PassEntry,
    PositionEncoding,
    RotaryTables,
    StateRequest,
    TensorSpec,
    build_part,
    register_part,
    registered_kinds,
)
from . import attention, block, embedding, entry, feedforward, latent, norm, recurrent, rope  # noqa: F401
