"""Parts a model is assembled from.  Importing the package registers the built-in ones."""
from . import (attention, block, delta, experts, latent, linear_attention, memory, mlp, norm, rope, side_by_side,  # noqa: F401
               token_side)  # noqa: F401
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, BranchSink, BranchTerms, OwedRows, Part, ResidualStream,
                   ScaleShape, StepContext, StepShape, StreamJoin, plain_rows,
                   build_part, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position_encoding)
from .block import build_block
from .linear import Linear
