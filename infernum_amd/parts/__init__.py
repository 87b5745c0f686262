"""Parts a decoder is put together from; importing this registers the built-in kinds."""
from .base import (Block, CacheSpec, CacheView, Embedding, FeedForward, Head, LayerSpec, Mixer, ModelSpec, Norm, PageTensor, Part,
                   PartSpec, PositionEncoding, QKTransform, Runtime, ScheduleEntry, StateSpec, StepContext, WeightSpec,
                   block_factory, make_part, part_kinds, register_part)
from . import (attention, block, branch_gate, conv_attention, embedding, gla, hgrn2, latent_attention, mamba2, mlp, moe,  # noqa: F401
               pooled_attention, rmsnorm, rope, sigmoid_attention, stream_in, token_side)  # noqa: F401  (registration)
from .linear import linear
