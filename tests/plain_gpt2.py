"""A plain, slow GPT-2: whole sequences, no cache, float64, one function a part.

Written from the reference's formulas (each function cites where); it shares
no code with `liyab_amd`: it reads the model folder with the `safetensors`
package and computes with numpy. Weights are used as stored (bfloat16
matrices are exact in float64); `round_weights_to_bf16` gives what the
bfloat16 path's matrices hold when the file stores float32.
"""

from __future__ import annotations

import json
import math
import os

import numpy as np


# ---------------------------------------------------------------------------
# reading a model folder
# ---------------------------------------------------------------------------
def read_model(model_dir):
    """(config dict, {name: float64 array}) with names stripped of 'transformer.'."""
    import torch
    from safetensors import safe_open

    with open(os.path.join(model_dir, "config.json")) as f:
        config = json.load(f)
    tensors = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            bare = name[len("transformer."):] if name.startswith("transformer.") else name
            tensors[bare] = t.to(torch.float64).numpy()
    return config, tensors


def round_to_bf16(a):
    """float64 -> nearest bfloat16 (ties to even) -> float64."""
    f = np.asarray(a, dtype=np.float32)
    u = f.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def round_weights_to_bf16(tensors):
    """Matrices (2-D) rounded to bfloat16, vectors untouched."""
    return {k: (round_to_bf16(v) if v.ndim >= 2 else v) for k, v in tensors.items()}


# ---------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------
def layer_norm(x, w, b, eps):
    """(x - mean) / sqrt(var + eps) * w + b, biased variance, over the last axis.
    Reference: layernorm, src/core/transformer.cpp:77-106."""
    mean = x.mean(axis=-1, keepdims=True)
    dev = x - mean
    var = (dev * dev).mean(axis=-1, keepdims=True)
    y = dev * (1.0 / np.sqrt(var + eps))
    if w is not None:
        y = y * w
    if b is not None:
        y = y + b
    return y


def gelu_tanh(x):
    """0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))).
    Reference: gelu_tanh, src/core/transformer.cpp:123-130."""
    return 0.5 * x * (1.0 + np.tanh(0.7978845608028654 * (x + 0.044715 * x * x * x)))


def gelu_erf(x):
    """0.5 x (1 + erf(x / sqrt 2)). Reference: gelu_erf, src/core/transformer.cpp:134-142."""
    erf = np.vectorize(math.erf, otypes=[np.float64])
    return 0.5 * x * (1.0 + erf(x * 0.70710678118654752440))


ACTIVATIONS = {"gelu_new": gelu_tanh, "gelu_pytorch_tanh": gelu_tanh, "gelu": gelu_erf}


def embed(wte, wpe, ids, positions):
    """x[t] = wte[id_t] + wpe[pos_t].
    Reference: embed, src/core/transformer.cpp:5495-5512; add_positions :2791-2808."""
    return wte[np.asarray(ids)] + wpe[np.asarray(positions)]


def qkv_projection(h, c_attn_w, c_attn_b):
    """qkv = h . W + b with W stored [d, 3d]; split [q | k | v] at d and 2d.
    Reference: project_fused_qkv, src/core/transformer.cpp:2657-2673; the fused bias is
    split the same way, :1263-1273, and added after the product, :3089-3101."""
    qkv = h @ c_attn_w + c_attn_b
    d = h.shape[-1]
    return qkv[:, :d], qkv[:, d:2 * d], qkv[:, 2 * d:]


def causal_attention(q, k, v, n_head, scale, window=0):
    """Per head: s_j = (k_j . q) * scale for j <= pos (own position included), softmax with the
    maximum subtracted, o = sum_j p_j v_j / sum_j p_j.
    Reference: attention, src/core/transformer.cpp:2162-2453 (scores :2303-2313, softmax
    :2327-2341, values :2344-2358, merge :2367-2385); a window sees [pos - window + 1, pos],
    :2155-2157."""
    T, d = q.shape
    hd = d // n_head
    out = np.zeros_like(q)
    for h in range(n_head):
        sl = slice(h * hd, (h + 1) * hd)
        for t in range(T):
            first = max(0, t - window + 1) if window > 0 else 0
            s = (k[first:t + 1, sl] @ q[t, sl]) * scale
            p = np.exp(s - s.max())
            out[t, sl] = (p[:, None] * v[first:t + 1, sl]).sum(axis=0) / p.sum()
    return out


def attention_scale(config, layer):
    """1/sqrt(head size) (src/compat/architecture.cpp:975-985, computed as 1.0f / sqrtf(hd));
    config.json's scale_attn_by_inverse_layer_idx divides it by layer + 1 and
    scale_attn_weights = false leaves 1 (both beside the reference, which has a per-block
    scale slot only, :1094)."""
    hd = config["n_embd"] // config["n_head"]
    s = 1.0 / math.sqrt(hd) if config.get("scale_attn_weights", True) else 1.0
    if config.get("scale_attn_by_inverse_layer_idx", False):
        s /= layer + 1
    return s


def attention_part(h, tensors, prefix, n_head, scale):
    """QKV -> attention -> output projection a = att . Wo + bo.
    Reference: attention_mixer, src/core/transformer.cpp:3083-3140."""
    q, k, v = qkv_projection(h, tensors[prefix + ".c_attn.weight"], tensors[prefix + ".c_attn.bias"])
    att = causal_attention(q, k, v, n_head, scale)
    return att @ tensors[prefix + ".c_proj.weight"] + tensors[prefix + ".c_proj.bias"]


def mlp_part(h, tensors, prefix, activation):
    """m = act(h . Wup + b_up) . Wdown + b_down.
    Reference: dense_ffn, FfnKind::Ungated, src/core/transformer.cpp:4903-4913."""
    inner = activation(h @ tensors[prefix + ".c_fc.weight"] + tensors[prefix + ".c_fc.bias"])
    return inner @ tensors[prefix + ".c_proj.weight"] + tensors[prefix + ".c_proj.bias"]


def block(x, tensors, config, layer):
    """x += attn(ln_1(x)); x += mlp(ln_2(x)).
    Reference: run_block, src/core/transformer.cpp:5514-5726 (norm :5565-5577, residual
    :5647, norm :5663-5666, residual :5692)."""
    p = f"h.{layer}"
    eps = config.get("layer_norm_epsilon", 1e-5)
    act = ACTIVATIONS[config.get("activation_function", "gelu_new")]
    h = layer_norm(x, tensors[p + ".ln_1.weight"], tensors[p + ".ln_1.bias"], eps)
    x = x + attention_part(h, tensors, p + ".attn", config["n_head"], attention_scale(config, layer))
    h = layer_norm(x, tensors[p + ".ln_2.weight"], tensors[p + ".ln_2.bias"], eps)
    return x + mlp_part(h, tensors, p + ".mlp", act)


def lm_head(x, tensors, config):
    """logits = ln_f(x) . wte^T (tied head; no bias, no scale).
    Reference: compute_logits, src/core/transformer.cpp:2622-2638; tie :1100-1104."""
    h = layer_norm(x, tensors["ln_f.weight"], tensors["ln_f.bias"], config.get("layer_norm_epsilon", 1e-5))
    w = tensors["wte.weight"] if config.get("tie_word_embeddings", True) else tensors["lm_head.weight"]
    return h @ w.T


def forward(config, tensors, ids, first_position=0):
    """Logits [T, vocab] (float64) of one whole sequence.
    Reference: Transformer::forward, src/core/transformer.cpp:6246-6258, 6284-6292."""
    ids = list(ids)
    x = embed(tensors["wte.weight"], tensors["wpe.weight"], ids, range(first_position, first_position + len(ids)))
    for layer in range(config["n_layer"]):
        x = block(x, tensors, config, layer)
    return lm_head(x, tensors, config)


# ---------------------------------------------------------------------------
# sampling
# ---------------------------------------------------------------------------
def probabilities(logits, temperature, top_k=0, top_p=1.0):
    """Temperature -> top-k -> top-p -> renormalise; one-hot at the first maximum when greedy.
    Reference: Sampler::probabilities, src/core/sampling.cpp:16-63. Ties in the descending
    order go by ascending id."""
    logits = np.asarray(logits, dtype=np.float32)
    n = logits.size
    probs = np.zeros(n, dtype=np.float64)
    if temperature <= 0:
        probs[int(np.argmax(logits))] = 1.0
        return probs
    order = sorted(range(n), key=lambda i: (-float(logits[i]), i))
    if 0 < top_k < n:
        order = order[:top_k]
    inv_t = np.float32(1.0) / np.float32(temperature)
    mx = logits[order[0]]
    p = {i: float(np.exp((logits[i] - mx) * inv_t, dtype=np.float32)) for i in order}
    total = sum(p.values())
    keep = len(order)
    if top_p < 1.0:
        cum = 0.0
        for j, i in enumerate(order):
            cum += p[i]
            if cum >= float(np.float32(top_p)) * total:
                keep = j + 1
                break
    kept = order[:keep]
    s = sum(p[i] for i in kept)
    for i in kept:
        probs[i] = p[i] / s
    return probs


def sample(probs, u):
    """r = u * total; walk ids upwards subtracting p_i; first r < 0 wins; fallback: the last id
    with mass. Reference: Sampler::sample, src/core/sampling.cpp:65-79."""
    total = float(np.sum(probs))
    r = u * total
    for i, p in enumerate(probs):
        r -= p
        if r < 0.0:
            return i
    nz = np.nonzero(probs)[0]
    return int(nz[-1]) if len(nz) else 0


def uniform(seed, index):
    """The engine's per-token uniform number: splitmix64 of (seed, index), top 53 bits."""
    mask = (1 << 64) - 1
    z = (seed * 0x9E3779B97F4A7C15 + (index + 1) * 0xD1B54A32D192ED03) & mask
    z = (z + 0x9E3779B97F4A7C15) & mask
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & mask
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & mask
    z = z ^ (z >> 31)
    return (z >> 11) * (1.0 / (1 << 53))


def generate_greedy(config, tensors, prompt, n_new):
    """Greedy continuation by full recompute (the last token sampled is not run)."""
    ids = list(prompt)
    out = []
    for _ in range(n_new):
        if len(ids) >= config["n_positions"]:
            break
        nxt = int(np.argmax(forward(config, tensors, ids)[-1].astype(np.float32)))
        out.append(nxt)
        ids.append(nxt)
    return out
