"""Parts a decoder is put together from.  Importing the package registers the
kinds the library ships."""

from .base import (  # noqa: F401
    Block,
    FeedForward,
    KVRequest,
    Mixer,
    Norm,
    Part,
    PositionEncoding,
    RotaryTables,
    StateRequest,
    TensorSpec,
    build_part,
    register_part,
    registered_kinds,
)
from . import attention, block, embedding, feedforward, norm, rope  # noqa: F401
