from . import block, feedforward, mixer, norm, position  # noqa: F401  (register the built-in kinds)
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, KvNeed, Part, PartSpec, Registry, RowTiling,
                   StateNeed)
from .context import CacheView, EntryInfo, KvCacheView, StateCacheView, StepContext
from .model import DecoderModel, LayerRun, ModelSpec, default_schedule
