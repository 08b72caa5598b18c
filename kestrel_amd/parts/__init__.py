"""Parts a model is put together from; importing the package registers the built-in kinds."""

from . import (attention, branches, decayed_memory, differential_attention, experts, junction, latent_attention, learned_position, matrix_memory, mlp, norm,
               pair_embedding, rotary)  # noqa: F401  (registration)
from .base import (FeedForward, Junction, LayerCache, Mixer, Norm, Part, PositionEncoding, Rotation, SideLinear, build_part, known_kinds,
                   register_feed_forward, register_junction, register_mixer, register_norm, register_position)
from .block import ARRANGEMENTS, Block, register_arrangement
from .specs import (AttentionSpec, BranchesSpec, CacheSpec, ConcatLinearSpec, DenseFeedForwardSpec, DistanceBuckets, DistanceSlopes,
                    GatedFeedForwardSpec, LayerSpec, LearnedPositionSpec, MatrixMemorySpec, ModelPlan, NormSpec, ParamSpec,
                    PositionSpec, QKNorm, QueryGrowth, ScheduleEntry, StateSpec, ValueBlend, WavelengthScaling)

__all__ = [
    "ARRANGEMENTS", "AttentionSpec", "Block", "BranchesSpec", "CacheSpec", "DistanceBuckets", "GatedFeedForwardSpec", "MatrixMemorySpec",
    "QKNorm", "QueryGrowth", "ValueBlend", "WavelengthScaling", "ConcatLinearSpec", "DenseFeedForwardSpec", "DistanceSlopes",
    "FeedForward", "Junction", "LayerCache", "LearnedPositionSpec", "register_junction",
    "LayerSpec", "Mixer", "ModelPlan", "Norm", "NormSpec", "ParamSpec", "Part", "PositionEncoding", "PositionSpec",
    "Rotation", "ScheduleEntry", "SideLinear", "StateSpec", "build_part", "known_kinds", "register_arrangement", "register_feed_forward",
    "register_mixer", "register_norm", "register_position",
]
