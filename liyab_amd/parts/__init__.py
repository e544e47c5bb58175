"""Model parts: mixers, feed-forwards, norms, position encodings, blocks."""

from .base import GroupStep, PartStepPlan, StepContext, StepFacts, StepHost, Workspace  # noqa: F401
from .registry import (  # noqa: F401
    build_part,
    find_part,
    register_block,
    register_embedding,
    register_ffn,
    register_head,
    register_mixer,
    register_norm,
    register_position,
)
from .norms import Normed, as_tensor  # noqa: F401
from . import attention, block, embeddings, feedforward, head, norms  # noqa: F401  (register themselves)
