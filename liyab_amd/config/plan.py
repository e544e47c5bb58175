"""The model plan: what an architecture's configuration turns into.

A plan is plain data. It lists the parts of each layer (mixer, feed-forward,
norms, position encoding) with their sizes and constants, the tensors each
part reads, and the order in which layers run. The engine builds parts from
a plan through the part registries and never looks at the architecture's
name again. The reference does the same with `ModelConfig` + one `BlockPlan`
per block (`src/compat/architecture.h:282-380, 452-630`): per-block mixer
kind, feed-forward kind, head counts, width and attention scale.

Every spec class carries a `kind` string; a registry maps the kind to the
part's class (`liyab_amd.parts.registry`). New kinds need no change here:
any dataclass with a `kind` attribute can stand in a `LayerSpec`.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional, Sequence


@dataclass(frozen=True)
class Init:
    """How the random-weights mode draws a tensor: N(mean, std)."""

    std: float
    mean: float = 0.0


@dataclass(frozen=True)
class TensorSource:
    """Where a part's tensor lives in the weights file.

    `layout` says how a matrix is stored: "out_in" = row per output feature
    (the reference's and this engine's working layout: `y = x . W^T`,
    `include/liyab/backend.h:35`), "in_out" = row per input feature (GPT-2's
    four projection matrices). The loader brings every matrix to "out_in".
    `init` is the distribution the random-weights mode draws the tensor from
    (None: N(0, 0.02)).
    """

    name: str
    layout: str = "out_in"
    required: bool = True
    init: Optional[Init] = None


@dataclass(frozen=True)
class NormSpec:
    kind: str  # "layernorm"
    width: int
    eps: float
    tensors: dict = field(default_factory=dict)  # "weight", "bias"


@dataclass(frozen=True)
class TokenEmbeddingSpec:
    kind: str  # "token_embedding"
    vocab_size: int
    width: int
    scale: float
    tensors: dict = field(default_factory=dict)  # "table"


@dataclass(frozen=True)
class PositionSpec:
    """A position encoding. `where` = "residual" (added to the embeddings, as learned
    positions are: the model's `residual_position`) or "mixer" (applied to queries and keys
    inside a mixer: that mixer's `position` field; the part then has `rotate(q, k, ctx)`)."""

    kind: str  # "learned_positions" | "none"
    where: str
    max_positions: int
    width: int
    tensors: dict = field(default_factory=dict)  # "table"


@dataclass(frozen=True)
class AttentionSpec:
    kind: str  # "attention"
    width: int
    n_head: int
    n_kv_head: int
    head_dim: int
    scale: float  # multiplies q.k before the softmax
    window: int  # 0 = every earlier position
    tensors: dict = field(default_factory=dict)  # qkv_weight, qkv_bias, out_weight, out_bias
    # a position encoding that acts on queries and keys (a spec with a `kind` of the position
    # registry and where = "mixer"), applied after the projection and before keys go to the cache
    position: Any = None


@dataclass(frozen=True)
class DenseFFNSpec:
    kind: str  # "dense_ffn"
    width: int
    inner: int
    activation: str  # "gelu_tanh" | "gelu_erf"
    tensors: dict = field(default_factory=dict)  # up_weight, up_bias, down_weight, down_bias


@dataclass(frozen=True)
class LayerSpec:
    """One block: which parts it has and how they are arranged.

    arrangement "pre_norm": x += mixer(norm_mixer(x)); x += ffn(norm_ffn(x)).
    """

    mixer: Any
    ffn: Any
    norm_mixer: Any
    norm_ffn: Any
    arrangement: str = "pre_norm"


@dataclass(frozen=True)
class OrderEntry:
    """One entry of the run order. `layer` indexes `ModelPlan.layers`;
    `cache_of` names the layer whose cache this run reads and writes
    (itself unless another layer's cache is shared)."""

    layer: int
    cache_of: Optional[int] = None
    writes_cache: bool = True

    @property
    def cache_layer(self) -> int:
        return self.layer if self.cache_of is None else self.cache_of


@dataclass(frozen=True)
class HeadSpec:
    kind: str  # "lm_head"
    width: int
    vocab_size: int
    logit_scale: float
    tensors: dict = field(default_factory=dict)  # "weight" (may name the embedding table), "bias"


@dataclass(frozen=True)
class ModelPlan:
    architecture: str
    width: int
    vocab_size: int
    max_positions: int
    embedding: TokenEmbeddingSpec
    residual_position: Optional[PositionSpec]
    layers: Sequence[LayerSpec]
    order: Sequence[OrderEntry]
    final_norm: Any
    head: HeadSpec
    # tensor-name patterns (fnmatch) that a file may hold and the engine ignores
    ignorable: Sequence[str] = ()
    # prefixes that may stand before every tensor name in a file
    name_prefixes: Sequence[str] = ("",)
    eos_token_id: Optional[int] = None
