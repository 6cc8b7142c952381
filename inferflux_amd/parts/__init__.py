"""Parts a model is assembled from.  Importing the package registers the built-in parts."""
from . import attention, block, embedding, ffn, norm, position  # noqa: F401
from .base import (Block, FeedForward, LayerCache, Mixer, MixerBinding, Norm, Part, build_part,
                   register_part, registered_parts)
from .plan import (CacheSpec, LayerSpec, ModelPlan, ParamSpec, PartSpec, ScheduleEntry, StateSpec)
from .position import PositionEncoding
