"""Parts a model is put together from.  Importing the package registers the built-in kinds."""
from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, LOGIT_STEPS, MATRIX, MIXERS, NORMS, POSITION_ENCODINGS, TABLE,
                   VECTOR32, Block, BuildEnv, CacheNeed, Embedding, FeedForward, KVNeed, LayerCache, LogitsStep, Mixer,
                   Norm, Part, PartSpec, PositionEncoding, Registry, StateNeed, StepContext, TensorSpec, Workspace,
                   build_part, project)
from . import attention, block, embedding, feedforward, norms, rope  # noqa: F401  (registration)

__all__ = [
    "BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "LOGIT_STEPS", "MATRIX", "MIXERS", "NORMS", "POSITION_ENCODINGS", "TABLE",
    "VECTOR32", "Block", "BuildEnv", "CacheNeed", "Embedding", "FeedForward", "KVNeed", "LayerCache", "LogitsStep",
    "Mixer", "Norm", "Part", "PartSpec", "PositionEncoding", "Registry", "StateNeed", "StepContext", "TensorSpec",
    "Workspace", "build_part", "project",
]
