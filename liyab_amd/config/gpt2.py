"""GPT-2's typed configuration, read from its own config.json keys.

Key names are those of the GPT-2 configuration the reference's conformance
record holds (`docs/validation/models-stage1/conformance.json:546-583`).
The reference itself reads the same facts from GGUF metadata
(`src/compat/architecture.cpp:588-600, 699-708, 798-805`) and fixes the rest
in its registry row `gpt2`: LayerNorm, no rotary encoding, tanh GELU, learned
positions, fused QKV, tied output (`src/compat/architecture.cpp:81-88`).
`activation_function`, `scale_attn_by_inverse_layer_idx`, `scale_attn_weights`
and `n_inner = null -> 4 n_embd` have no counterpart there and follow the
configuration's own meaning.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

from ..errors import InvalidModel, Unsupported
from .plan import (
    AttentionSpec,
    DenseFFNSpec,
    HeadSpec,
    Init,
    LayerSpec,
    ModelPlan,
    NormSpec,
    OrderEntry,
    PositionSpec,
    TensorSource,
    TokenEmbeddingSpec,
)
from .registry import register_architecture

_ACTIVATIONS = {
    "gelu_new": "gelu_tanh",
    "gelu_pytorch_tanh": "gelu_tanh",
    "gelu": "gelu_erf",
}

_LIMIT = 1 << 24  # the reference's bound on counts, src/compat/architecture.cpp:590


def _require_int(raw: dict, key: str, *, fallback: Optional[str] = None) -> int:
    v = raw.get(key)
    if v is None and fallback is not None:
        v = raw.get(fallback)
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0 or v > _LIMIT:
        raise InvalidModel(f"missing or invalid {key}")
    return v


def _bool(raw: dict, key: str, default: bool) -> bool:
    v = raw.get(key, default)
    if v is None:
        return default
    if not isinstance(v, bool):
        raise InvalidModel(f"invalid {key}: expected true or false")
    return v


@dataclass(frozen=True)
class GPT2Config:
    n_layer: int
    n_embd: int
    n_head: int
    n_inner: int
    vocab_size: int
    n_positions: int
    layer_norm_epsilon: float
    activation_function: str
    scale_attn_weights: bool
    scale_attn_by_inverse_layer_idx: bool
    tie_word_embeddings: bool
    eos_token_id: Optional[int]
    bos_token_id: Optional[int]

    architecture = "GPT2LMHeadModel"

    @property
    def head_dim(self) -> int:
        return self.n_embd // self.n_head

    @classmethod
    def from_json(cls, raw: dict) -> "GPT2Config":
        n_layer = _require_int(raw, "n_layer")
        n_embd = _require_int(raw, "n_embd")
        n_head = _require_int(raw, "n_head")
        if n_embd % n_head != 0:
            raise InvalidModel(f"invalid n_head: {n_head} does not divide n_embd {n_embd}")
        n_inner = raw.get("n_inner")
        if n_inner is None:
            n_inner = 4 * n_embd
        elif isinstance(n_inner, bool) or not isinstance(n_inner, int) or n_inner <= 0 or n_inner > _LIMIT:
            raise InvalidModel("missing or invalid n_inner")
        vocab_size = _require_int(raw, "vocab_size")
        n_positions = _require_int(raw, "n_positions", fallback="n_ctx")
        eps = raw.get("layer_norm_epsilon", 1e-5)
        if isinstance(eps, bool) or not isinstance(eps, (int, float)) or not math.isfinite(eps) or eps < 0:
            raise InvalidModel("invalid norm epsilon")  # src/compat/architecture.cpp:803-805
        act = raw.get("activation_function", "gelu_new")
        if act not in _ACTIVATIONS:
            raise Unsupported(
                f"activation_function '{act}' is not supported (supported: {','.join(sorted(_ACTIVATIONS))})"
            )
        if _bool(raw, "add_cross_attention", False):
            raise Unsupported("add_cross_attention is not supported")
        for key in ("eos_token_id", "bos_token_id"):
            v = raw.get(key)
            if v is not None and (isinstance(v, bool) or not isinstance(v, int)):
                raise InvalidModel(f"invalid {key}")
        return cls(
            n_layer=n_layer,
            n_embd=n_embd,
            n_head=n_head,
            n_inner=n_inner,
            vocab_size=vocab_size,
            n_positions=n_positions,
            layer_norm_epsilon=float(eps),
            activation_function=act,
            scale_attn_weights=_bool(raw, "scale_attn_weights", True),
            scale_attn_by_inverse_layer_idx=_bool(raw, "scale_attn_by_inverse_layer_idx", False),
            tie_word_embeddings=_bool(raw, "tie_word_embeddings", True),
            eos_token_id=raw.get("eos_token_id"),
            bos_token_id=raw.get("bos_token_id"),
        )

    def to_json(self) -> dict:
        return {
            "architectures": [self.architecture],
            "model_type": "gpt2",
            "n_layer": self.n_layer,
            "n_embd": self.n_embd,
            "n_head": self.n_head,
            "n_inner": self.n_inner,
            "vocab_size": self.vocab_size,
            "n_positions": self.n_positions,
            "n_ctx": self.n_positions,
            "layer_norm_epsilon": self.layer_norm_epsilon,
            "activation_function": self.activation_function,
            "scale_attn_weights": self.scale_attn_weights,
            "scale_attn_by_inverse_layer_idx": self.scale_attn_by_inverse_layer_idx,
            "tie_word_embeddings": self.tie_word_embeddings,
            "eos_token_id": self.eos_token_id,
            "bos_token_id": self.bos_token_id,
        }

    def attention_scale(self, layer: int) -> float:
        """What multiplies q.k in `layer` (0-based). The reference's default is
        1/sqrt(head size) (`src/compat/architecture.cpp:975-985`) in a per-block
        slot (`:1094`); the inverse-layer factor divides it by layer + 1."""
        s = 1.0 / math.sqrt(self.head_dim) if self.scale_attn_weights else 1.0
        if self.scale_attn_by_inverse_layer_idx:
            s /= float(layer + 1)
        return s

    def plan(self) -> ModelPlan:
        d, F, V = self.n_embd, self.n_inner, self.vocab_size
        eps = self.layer_norm_epsilon
        # What the random-weights mode draws: embeddings and the products into a layer N(0, 0.02), the
        # two products back to the stream N(0, 0.02 / sqrt(2 n_layer)), biases N(0, 0.02), norm weights
        # 1 + N(0, 0.05) and norm biases N(0, 0.02). Norm weights away from 1 and biases away from 0
        # make a norm or a bias applied in the wrong place visible (tools/reference_trace.py:424-437
        # argues the same for its own random checkpoints).
        wide, bias = Init(0.02), Init(0.02)
        back = Init(0.02 / math.sqrt(2.0 * self.n_layer))

        def norm(prefix: str) -> NormSpec:
            return NormSpec(
                kind="layernorm",
                width=d,
                eps=eps,
                tensors={
                    "weight": TensorSource(prefix + ".weight", init=Init(0.05, 1.0)),
                    "bias": TensorSource(prefix + ".bias", init=bias),
                },
            )

        layers = []
        for i in range(self.n_layer):
            p = f"h.{i}"
            mixer = AttentionSpec(
                kind="attention",
                width=d,
                n_head=self.n_head,
                n_kv_head=self.n_head,
                head_dim=self.head_dim,
                scale=self.attention_scale(i),
                window=0,
                tensors={
                    "qkv_weight": TensorSource(p + ".attn.c_attn.weight", layout="in_out", init=wide),
                    "qkv_bias": TensorSource(p + ".attn.c_attn.bias", init=bias),
                    "out_weight": TensorSource(p + ".attn.c_proj.weight", layout="in_out", init=back),
                    "out_bias": TensorSource(p + ".attn.c_proj.bias", init=bias),
                },
            )
            ffn = DenseFFNSpec(
                kind="dense_ffn",
                width=d,
                inner=F,
                activation=_ACTIVATIONS[self.activation_function],
                tensors={
                    "up_weight": TensorSource(p + ".mlp.c_fc.weight", layout="in_out", init=wide),
                    "up_bias": TensorSource(p + ".mlp.c_fc.bias", init=bias),
                    "down_weight": TensorSource(p + ".mlp.c_proj.weight", layout="in_out", init=back),
                    "down_bias": TensorSource(p + ".mlp.c_proj.bias", init=bias),
                },
            )
            layers.append(
                LayerSpec(mixer=mixer, ffn=ffn, norm_mixer=norm(p + ".ln_1"), norm_ffn=norm(p + ".ln_2"))
            )
        head_weight = "wte.weight" if self.tie_word_embeddings else "lm_head.weight"
        ignorable = ["h.*.attn.bias", "h.*.attn.masked_bias"]
        if self.tie_word_embeddings:
            ignorable.append("lm_head.weight")  # the same tensor as wte when tied
        return ModelPlan(
            architecture=self.architecture,
            width=d,
            vocab_size=V,
            max_positions=self.n_positions,
            embedding=TokenEmbeddingSpec(
                kind="token_embedding",
                vocab_size=V,
                width=d,
                scale=1.0,
                tensors={"table": TensorSource("wte.weight", init=wide)},
            ),
            residual_position=PositionSpec(
                kind="learned_positions",
                where="residual",
                max_positions=self.n_positions,
                width=d,
                tensors={"table": TensorSource("wpe.weight", init=wide)},
            ),
            layers=layers,
            order=[OrderEntry(layer=i) for i in range(self.n_layer)],
            final_norm=norm("ln_f"),
            head=HeadSpec(
                kind="lm_head",
                width=d,
                vocab_size=V,
                logit_scale=1.0,
                tensors={"weight": TensorSource(head_weight, init=wide), "bias": TensorSource("lm_head.bias", required=False)},
            ),
            ignorable=tuple(ignorable),
            name_prefixes=("", "transformer."),
            eos_token_id=self.eos_token_id,
        )


register_architecture("GPT2LMHeadModel", GPT2Config, model_types=["gpt2"])
