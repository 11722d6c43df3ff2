from .spec import PartSpec, LayerSpec, ScheduleEntry, ModelSpec
from .base import (Part, Mixer, PositionEncoding, CacheNeed, StepPlan, BatchInfo, register_part, build_part,
                   CATEGORIES)

__all__ = ["PartSpec", "LayerSpec", "ScheduleEntry", "ModelSpec", "Part", "Mixer", "PositionEncoding",
           "CacheNeed", "StepPlan", "BatchInfo", "register_part", "build_part", "CATEGORIES"]
