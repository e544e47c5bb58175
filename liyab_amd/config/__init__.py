"""Typed configurations and the architecture registry."""

from .plan import (  # noqa: F401
    AttentionSpec,
    DenseFFNSpec,
    HeadSpec,
    LayerSpec,
    ModelPlan,
    NormSpec,
    OrderEntry,
    PositionSpec,
    TensorSource,
    TokenEmbeddingSpec,
)
from .registry import (  # noqa: F401
    architecture_name_of,
    config_from_dict,
    find_architecture,
    load_config,
    register_architecture,
    supported_architectures,
)
from .gpt2 import GPT2Config  # noqa: F401  (registers itself)
