"""Parts a decoder is put together from; importing this registers the built-in kinds."""
from .base import (Block, CacheSpec, CacheView, Embedding, FeedForward, Head, LayerSpec, Mixer, ModelSpec, Norm, PageTensor, Part,
                   PartSpec, PositionEncoding, QKTransform, Runtime, ScheduleEntry, StateSpec, StepContext, WeightSpec,
                   block_factory, make_part, part_kinds, register_part)
from . import attention, block, embedding, mlp, rmsnorm, rope  # noqa: F401  (registration)
from .linear import linear
