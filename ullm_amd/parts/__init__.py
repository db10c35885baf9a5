"""Parts a layer is put together from.  Importing the package registers the built-in parts."""
from .base import (Block, CacheNeed, CacheRows, Embedder, FeedForward, GroupView, KVNeed, LayerCache, Mixer, Norm, NormedBranch, Part, PartEnv,
                   PendingNorm, PositionEncoding, StateNeed, StepContext, StepPlan, StepShape, StreamsBranch, WeightDecl, build_part,
                   register_part, registered_parts, walk, cache_needs_of)
from . import norm, position, attention, feedforward, block, embedding, ssm, moe, latent, decay  # noqa: F401  (registration)

__all__ = ["Block", "Embedder", "NormedBranch", "CacheNeed", "CacheRows", "StepPlan", "StepShape", "FeedForward", "GroupView", "KVNeed", "LayerCache", "Mixer", "Norm", "Part",
           "PartEnv", "PendingNorm", "PositionEncoding", "StreamsBranch", "StateNeed", "StepContext", "WeightDecl", "build_part",
           "register_part", "registered_parts", "walk", "cache_needs_of"]
