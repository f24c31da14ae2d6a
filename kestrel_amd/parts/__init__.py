"""Parts a model is put together from; importing the package registers the built-in kinds."""

from . import attention, mlp, norm, rotary  # noqa: F401  (registration)
from .base import (FeedForward, LayerCache, Mixer, Norm, Part, PositionEncoding, Rotation, SideLinear, build_part, known_kinds,
                   register_feed_forward, register_mixer, register_norm, register_position)
from .block import ARRANGEMENTS, Block, register_arrangement
from .specs import (AttentionSpec, CacheSpec, DenseFeedForwardSpec, LayerSpec, ModelPlan, NormSpec, ParamSpec,
                    PositionSpec, ScheduleEntry, StateSpec)

__all__ = [
    "ARRANGEMENTS", "AttentionSpec", "Block", "CacheSpec", "DenseFeedForwardSpec", "FeedForward", "LayerCache",
    "LayerSpec", "Mixer", "ModelPlan", "Norm", "NormSpec", "ParamSpec", "Part", "PositionEncoding", "PositionSpec",
    "Rotation", "ScheduleEntry", "SideLinear", "StateSpec", "build_part", "known_kinds", "register_arrangement", "register_feed_forward",
    "register_mixer", "register_norm", "register_position",
]
