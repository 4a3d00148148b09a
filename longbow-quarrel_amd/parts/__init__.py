"""Parts a model is put together from.  Importing the package registers the built-in kinds."""
from .base import (BLOCKS, FEED_FORWARDS, MATRIX, MIXERS, NORMS, POSITION_ENCODINGS, TABLE, VECTOR32,
                   Block, BuildEnv, FeedForward, KVNeed, LayerCache, Mixer, Norm, Part, PartSpec,
                   PositionEncoding, Registry, StateNeed, StepContext, TensorSpec, Workspace, build_part, project)
from . import attention, block, feedforward, norms, rope  # noqa: F401  (registration)

__all__ = [
    "BLOCKS", "FEED_FORWARDS", "MATRIX", "MIXERS", "NORMS", "POSITION_ENCODINGS", "TABLE", "VECTOR32",
    "Block", "BuildEnv", "FeedForward", "KVNeed", "LayerCache", "Mixer", "Norm", "Part", "PartSpec",
    "PositionEncoding", "Registry", "StateNeed", "StepContext", "TensorSpec", "Workspace", "build_part", "project",
]
