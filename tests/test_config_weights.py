"""Configuration, registry, safetensors and the weights' one error (no GPU)."""

import json
import os
import struct

import numpy as np
import pytest
import torch

from conftest import CONFIG_A, CONFIG_B
from liyab_amd import InvalidModel, Unsupported
from liyab_amd.config import GPT2Config, config_from_dict, find_architecture, load_config, supported_architectures
from liyab_amd.models.decoder import DecoderModel
from liyab_amd.weights import SafetensorsFile, WeightStore, random_tensors, write_random_model, write_safetensors


def test_config_reads_every_key():
    a = config_from_dict(dict(CONFIG_A))
    assert isinstance(a, GPT2Config)
    assert (a.n_layer, a.n_embd, a.n_head, a.n_inner, a.vocab_size, a.n_positions) == (2, 64, 4, 256, 512, 128)
    assert a.head_dim == 16 and a.layer_norm_epsilon == 1e-5 and a.activation_function == "gelu_new"
    b = config_from_dict(dict(CONFIG_B))
    assert (b.n_layer, b.n_embd, b.n_head, b.n_inner, b.vocab_size, b.n_positions) == (3, 96, 3, 320, 1000, 256)
    assert b.head_dim == 32 and b.layer_norm_epsilon == 1e-6 and b.scale_attn_by_inverse_layer_idx
    assert b.attention_scale(0) == pytest.approx(32 ** -0.5) and b.attention_scale(2) == pytest.approx(32 ** -0.5 / 3)
    pa, pb = a.plan(), b.plan()
    assert len(pa.layers) == 2 and len(pb.layers) == 3 and [e.layer for e in pb.order] == [0, 1, 2]
    assert pa.layers[0].ffn.activation == "gelu_tanh" and pb.layers[0].ffn.activation == "gelu_erf"
    assert pb.layers[2].mixer.scale == pytest.approx(32 ** -0.5 / 3) and pb.layers[1].ffn.inner == 320
    assert pa.layers[0].norm_mixer.eps == 1e-5 and pb.final_norm.eps == 1e-6
    assert pa.head.tensors["weight"].name == "wte.weight"  # tied


def test_config_defaults_and_fallbacks():
    raw = {"model_type": "gpt2", "n_layer": 1, "n_embd": 32, "n_head": 2, "vocab_size": 50, "n_ctx": 64}
    c = config_from_dict(raw)
    assert c.n_positions == 64 and c.n_inner == 128 and c.layer_norm_epsilon == 1e-5
    assert c.activation_function == "gelu_new" and c.tie_word_embeddings and c.scale_attn_weights
    assert config_from_dict(dict(raw, scale_attn_weights=False)).attention_scale(0) == 1.0
    assert config_from_dict(c.to_json()) == c


@pytest.mark.parametrize("change,exc,text", [
    ({"n_layer": None}, InvalidModel, "missing or invalid n_layer"),
    ({"n_embd": 0}, InvalidModel, "missing or invalid n_embd"),
    ({"n_head": 5}, InvalidModel, "does not divide"),
    ({"vocab_size": "x"}, InvalidModel, "missing or invalid vocab_size"),
    ({"n_inner": -3}, InvalidModel, "missing or invalid n_inner"),
    ({"layer_norm_epsilon": -1.0}, InvalidModel, "invalid norm epsilon"),
    ({"layer_norm_epsilon": float("nan")}, InvalidModel, "invalid norm epsilon"),
    ({"activation_function": "relu"}, Unsupported, "activation_function 'relu'"),
    ({"scale_attn_by_inverse_layer_idx": 1}, InvalidModel, "scale_attn_by_inverse_layer_idx"),
    ({"add_cross_attention": True}, Unsupported, "add_cross_attention"),
])
def test_config_errors_name_the_key(change, exc, text):
    with pytest.raises(exc, match=text):
        config_from_dict(dict(CONFIG_A, **change))


def test_registry_names_what_is_supported(tmp_path):
    assert find_architecture("GPT2LMHeadModel") is GPT2Config
    with pytest.raises(Unsupported, match=r"architecture 'LlamaForCausalLM' is not supported yet \(supported: .*GPT2LMHeadModel"):
        config_from_dict({"architectures": ["LlamaForCausalLM"]})
    with pytest.raises(Unsupported, match="'mamba'"):
        config_from_dict({"model_type": "mamba"})
    with pytest.raises(InvalidModel, match="neither"):
        config_from_dict({"n_layer": 2})
    assert "GPT2LMHeadModel" in supported_architectures()
    with pytest.raises(InvalidModel, match="config.json"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(InvalidModel, match="not valid JSON"):
        load_config(str(tmp_path))


def test_safetensors_round_trip_and_against_the_package(tmp_path):
    from safetensors.torch import load_file, save_file

    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int32).reshape(2, 3),
               "empty": torch.zeros(0, 4)}
    p = str(tmp_path / "x.safetensors")
    write_safetensors(p, tensors, {"k": "v"})
    f = SafetensorsFile(p)
    assert f.metadata == {"k": "v"}
    for k, v in tensors.items():
        assert f.entries[k].shape == tuple(v.shape) and torch.equal(f.tensor(k), v)
    theirs = load_file(p)  # the package reads what we wrote
    assert all(torch.equal(theirs[k], v) for k, v in tensors.items())
    p2 = str(tmp_path / "y.safetensors")
    save_file({k: v for k, v in tensors.items() if k != "empty"}, p2)  # and we read what it wrote
    g = SafetensorsFile(p2)
    assert all(torch.equal(g.tensor(k), tensors[k]) for k in g.entries)


def test_malformed_safetensors_are_refused(tmp_path):
    def write(name, header, data=b"", hlen=None):
        raw = json.dumps(header).encode() if not isinstance(header, bytes) else header
        p = tmp_path / name
        p.write_bytes(struct.pack("<Q", len(raw) if hlen is None else hlen) + raw + data)
        return str(p)

    with pytest.raises(InvalidModel, match="shorter"):
        (tmp_path / "s").write_bytes(b"abc")
        SafetensorsFile(str(tmp_path / "s"))
    with pytest.raises(InvalidModel, match="header length"):
        SafetensorsFile(write("h", {}, hlen=10**9))
    with pytest.raises(InvalidModel, match="malformed header"):
        SafetensorsFile(write("j", b"{nope}"))
    with pytest.raises(InvalidModel, match="unknown dtype"):
        SafetensorsFile(write("d", {"t": {"dtype": "F8_E9", "shape": [1], "data_offsets": [0, 1]}}, b"\0"))
    with pytest.raises(InvalidModel, match="do not fit"):
        SafetensorsFile(write("o", {"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, b"\0" * 8))
    with pytest.raises(InvalidModel, match="do not fit"):
        SafetensorsFile(write("z", {"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 16]}}, b"\0" * 16))
    with pytest.raises(InvalidModel, match="duplicate"):
        SafetensorsFile(write("u", b'{"t":{"dtype":"F32","shape":[1],"data_offsets":[0,4]},"t":{"dtype":"F32","shape":[1],"data_offsets":[0,4]}}', b"\0" * 4))
    with pytest.raises(InvalidModel, match="missing"):
        SafetensorsFile(str(tmp_path / "nothing.safetensors"))


def _build(tensors, cfg=CONFIG_A, dtype=torch.float32):
    plan = config_from_dict(dict(cfg)).plan()
    store = WeightStore(tensors, device="cpu", compute_dtype=dtype, name_prefixes=plan.name_prefixes, ignorable=plan.ignorable)
    model = DecoderModel(plan, store, dtype)
    store.finish()
    return model


def test_weights_load_by_name_with_dtypes_and_layouts():
    cfg = config_from_dict(dict(CONFIG_A))
    t = random_tensors(cfg, 0)
    t["h.0.attn.bias"] = torch.ones(1, 1, 8, 8)  # buffers a checkpoint may carry: ignored
    t["h.1.attn.masked_bias"] = torch.tensor(-1e4)
    t["lm_head.weight"] = t["wte.weight"]
    m = _build(t, dtype=torch.bfloat16)
    att = m.blocks[0].mixer
    assert att.qkv_weight.shape == (192, 64) and att.qkv_weight.dtype == torch.bfloat16  # [out, in]: transposed at load
    assert torch.equal(att.qkv_weight, t["h.0.attn.c_attn.weight"].t().to(torch.bfloat16))
    assert att.qkv_bias.dtype == torch.float32 and m.blocks[1].norm_ffn.weight.dtype == torch.float32
    assert m.head.weight.data_ptr() == m.embedding.table.data_ptr()  # tied: resident once
    m32 = _build({("transformer." + k): v for k, v in random_tensors(cfg, 0).items()})  # prefixed names
    assert m32.blocks[0].ffn.up_weight.dtype == torch.float32 and m32.blocks[0].ffn.up_weight.shape == (256, 64)
    # a file stored in bfloat16 runs on the 32-bit path too (exact upcast)
    bf = {k: (v.to(torch.bfloat16) if v.dim() == 2 else v) for k, v in random_tensors(cfg, 0).items()}
    m3 = _build(bf)
    assert m3.embedding.table.dtype == torch.float32
    assert torch.equal(m3.embedding.table, bf["wte.weight"].float())


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    cfg = config_from_dict(dict(CONFIG_A))
    t = random_tensors(cfg, 0)
    del t["h.1.ln_2.bias"], t["wpe.weight"]
    t["h.0.mlp.c_fc.weight"] = torch.zeros(256, 64)  # stored [out, in]: the wrong way round
    t["ln_f.weight"] = torch.zeros(65)
    t["h.0.attn.rotary.inv_freq"] = torch.zeros(8)
    t["h.1.ln_1.weight"] = torch.zeros(64, dtype=torch.int32)
    with pytest.raises(InvalidModel) as e:
        _build(t)
    msg = str(e.value)
    assert "missing tensors (2): " in msg and "'h.1.ln_2.bias'" in msg and "'wpe.weight'" in msg
    assert "tensor 'h.0.mlp.c_fc.weight' has shape [256, 64], expected [64, 256]" in msg
    assert "tensor 'ln_f.weight' has shape [65], expected [64]" in msg
    assert "unexpected tensors (1): 'h.0.attn.rotary.inv_freq'" in msg
    assert "tensor 'h.1.ln_1.weight' holds torch.int32" in msg


def test_untied_head_needs_its_tensor():
    cfg = config_from_dict(dict(CONFIG_A, tie_word_embeddings=False))
    t = random_tensors(cfg, 0)
    m = _build(t, cfg=dict(CONFIG_A, tie_word_embeddings=False))
    assert m.head.weight.data_ptr() != m.embedding.table.data_ptr()
    del t["lm_head.weight"]
    with pytest.raises(InvalidModel, match="lm_head.weight"):
        _build(t, cfg=dict(CONFIG_A, tie_word_embeddings=False))


def test_random_weights_mode_writes_a_folder(tmp_path):
    d1 = write_random_model(str(tmp_path / "m1"), dict(CONFIG_B), 2)
    d2 = write_random_model(str(tmp_path / "m2"), dict(CONFIG_B), 2)
    d3 = write_random_model(str(tmp_path / "m3"), dict(CONFIG_B), 3, dtype="bfloat16")
    assert sorted(os.listdir(d1)) == ["config.json", "model.safetensors"]
    assert load_config(d1) == config_from_dict(dict(CONFIG_B))
    f1, f2, f3 = (SafetensorsFile(os.path.join(d, "model.safetensors")) for d in (d1, d2, d3))
    assert set(f1.entries) == set(f2.entries) and len(f1.entries) == 2 + 12 * 3 + 2
    for k in f1.entries:
        assert torch.equal(f1.tensor(k), f2.tensor(k))  # the same seed gives the same bytes
    assert not torch.equal(f1.tensor("wte.weight"), f3.tensor("wte.weight").float())
    assert f3.tensor("wte.weight").dtype == torch.bfloat16 and f3.tensor("ln_f.weight").dtype == torch.float32
    assert f1.tensor("h.0.attn.c_attn.weight").shape == (96, 288) and f1.tensor("h.2.mlp.c_proj.weight").shape == (320, 96)
    w = f1.tensor("h.1.mlp.c_fc.weight").double()
    assert abs(w.std().item() - 0.02) < 2e-3 and abs(f1.tensor("h.0.ln_1.weight").mean().item() - 1.0) < 0.05
    assert abs(f1.tensor("h.1.attn.c_proj.weight").double().std().item() - 0.02 / (2 * 3) ** 0.5) < 1e-3


def test_random_weights_come_from_the_plan_not_from_an_architecture():
    """A plan nobody has registered as an architecture, with a part of its own: the
    random-weights mode draws exactly what its parts ask for, each tensor from the rule the
    plan gives with its name, in the layout the plan says the file holds; and a tensor's
    values depend on the seed and its name only."""
    from liyab_amd.config.plan import (HeadSpec, Init, LayerSpec, ModelPlan, NormSpec, OrderEntry, TensorSource,
                                       TokenEmbeddingSpec)
    from liyab_amd.parts.registry import register_mixer

    class Gate:  # a mixer that scales the stream by a learned vector and keeps nothing
        def __init__(self, spec, store, dtype):
            self.scale = store.fetch(spec.tensors["scale"], (spec.width,), "vector")
            self.mix = store.fetch(spec.tensors["mix"], (spec.width, 7), "matrix")
            self.extra = store.fetch(spec.tensors["extra"], (3,), "vector")  # optional, absent

        def cache_spec(self): return None
        def state_spec(self): return None

    register_mixer("test_gate", Gate)

    class GateSpec:
        kind = "test_gate"

        def __init__(self, layer, width):
            self.width = width
            self.tensors = {"scale": TensorSource(f"l.{layer}.scale", init=Init(0.5, 3.0)),
                            "mix": TensorSource(f"l.{layer}.mix", layout="in_out"),
                            "extra": TensorSource(f"l.{layer}.extra", required=False)}

    def toy(n_layer, d=12, V=40):
        emb = TokenEmbeddingSpec("token_embedding", V, d, 1.0, {"table": TensorSource("emb", init=Init(1.0))})
        layers = [LayerSpec(mixer=GateSpec(i, d), ffn=None, norm_mixer=None, norm_ffn=None) for i in range(n_layer)]
        return ModelPlan(architecture="toy", width=d, vocab_size=V, max_positions=64, embedding=emb, residual_position=None,
                         layers=layers, order=[OrderEntry(i) for i in range(n_layer)],
                         final_norm=NormSpec("layernorm", d, 1e-5, {"weight": TensorSource("out_norm.w", init=Init(0.05, 1.0))}),
                         head=HeadSpec("lm_head", d, V, 1.0, {"weight": TensorSource("emb")}))

    t2, t3 = random_tensors(toy(2), 9), random_tensors(toy(3), 9)
    assert sorted(t2) == ["emb", "l.0.mix", "l.0.scale", "l.1.mix", "l.1.scale", "out_norm.w"]
    assert t2["l.0.mix"].shape == (7, 12)  # stored [in, out], as the plan says
    assert abs(t2["l.1.scale"].mean().item() - 3.0) < 0.6 and abs(t2["emb"].std().item() - 1.0) < 0.15
    assert abs(t2["l.0.mix"].std().item() - 0.02) < 0.01  # no rule given: N(0, 0.02)
    for k in t2:
        assert torch.equal(t2[k], t3[k])  # another layer changes none of the others
    assert not torch.equal(t2["l.0.scale"], random_tensors(toy(2), 10)["l.0.scale"])
    assert not torch.equal(t2["l.0.scale"], t2["l.1.scale"])


def test_the_four_projection_matrices_share_one_stored_layout():
    """GPT-2's checkpoints hold c_attn, attn.c_proj, c_fc and mlp.c_proj under one rule: the
    reference's converter treats exactly these four suffixes in one branch
    (docs/validation/models-stage1/converter-classic.patch:14-20). Three of them show by their
    shapes which way round they are stored ([in, out]: c_attn is [d, 3d]); the square attn.c_proj
    cannot, and follows the rule of the other three. The loader refuses each of the three
    unambiguous ones when it is stored the other way round."""
    cfg = config_from_dict(dict(CONFIG_B))
    plan = cfg.plan()
    for layer in plan.layers:
        layouts = {layer.mixer.tensors["qkv_weight"].layout, layer.mixer.tensors["out_weight"].layout,
                   layer.ffn.tensors["up_weight"].layout, layer.ffn.tensors["down_weight"].layout}
        assert layouts == {"in_out"}
    for name, shape in (("h.0.attn.c_attn.weight", [96, 288]), ("h.1.mlp.c_fc.weight", [96, 320]),
                        ("h.2.mlp.c_proj.weight", [320, 96])):
        t = random_tensors(cfg, 1)
        assert list(t[name].shape) == shape
        t[name] = t[name].t().contiguous()
        with pytest.raises(InvalidModel, match=name.replace(".", r"\.")):
            _build(t, cfg=CONFIG_B)
