"""Parts a model is assembled from.  Importing the package registers the built-in ones."""
from . import attention, block, mlp, norm, rope  # noqa: F401
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, BranchSink, OwedRows, Part, ResidualStream,
                   ScaleShape, StepContext, StepShape, plain_rows,
                   build_part, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position_encoding)
from .block import build_block
from .linear import Linear
