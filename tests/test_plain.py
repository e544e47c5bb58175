"""What fixes the plain implementation beside the reference's text: special cases that
reduce to a library routine, invariants, and the constants the reference's files hold.
Each is chosen so that a plausible mistake fails it."""

import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_gpt2 as plain
from conftest import CONFIGS

RNG = np.random.default_rng(0)


def test_layer_norm_is_the_library_routine_with_biased_variance():
    x = RNG.standard_normal((5, 96)) * 3 + 1.5
    w, b = RNG.standard_normal(96), RNG.standard_normal(96)
    for eps in (1e-5, 1e-6):
        want = F.layer_norm(torch.tensor(x), (96,), torch.tensor(w), torch.tensor(b), eps).numpy()
        assert np.allclose(plain.layer_norm(x, w, b, eps), want, rtol=1e-12, atol=1e-12)
    # unbiased variance (d - 1) would differ by far more than rounding
    unbiased = (x - x.mean(-1, keepdims=True)) / np.sqrt(x.var(-1, ddof=1, keepdims=True) + 1e-5) * w + b
    assert np.abs(unbiased - plain.layer_norm(x, w, b, 1e-5)).max() > 1e-3


def test_layer_norm_invariants():
    x = RNG.standard_normal((3, 64))
    w, b = RNG.standard_normal(64), RNG.standard_normal(64)
    assert np.allclose(plain.layer_norm(x + 7.25, w, b, 1e-5), plain.layer_norm(x, w, b, 1e-5), atol=1e-9)
    y = plain.layer_norm(x, None, None, 1e-5)
    assert np.abs(y.mean(-1)).max() < 1e-12
    # eps matters on a low-variance row: 1e-5 and 1e-6 give measurably different results
    flat = 1.0 + 1e-3 * RNG.standard_normal((1, 64))
    assert np.abs(plain.layer_norm(flat, w, None, 1e-5) - plain.layer_norm(flat, w, None, 1e-6)).max() > 1e-2
    # the weight multiplies (not 1 + w) and the bias comes after it
    assert np.allclose(plain.layer_norm(x, np.zeros(64), b, 1e-5), np.broadcast_to(b, x.shape))


def test_gelu_forms_are_the_library_routines_and_differ():
    x = np.linspace(-6, 6, 1201)
    t = torch.tensor(x)
    assert np.allclose(plain.gelu_tanh(x), F.gelu(t, approximate="tanh").numpy(), atol=1e-12)
    assert np.allclose(plain.gelu_erf(x), F.gelu(t).numpy(), atol=1e-12)
    # the two forms differ by up to ~5e-4 near |x| = 2: the wrong one fails a 1e-5 check
    assert 1e-4 < np.abs(plain.gelu_tanh(x) - plain.gelu_erf(x)).max() < 1e-3
    for g in (plain.gelu_tanh, plain.gelu_erf):
        assert np.allclose(g(x) - g(-x), x, atol=1e-12)  # gelu(x) - gelu(-x) = x
        assert g(np.zeros(1))[0] == 0.0
    # the constants the reference writes out (src/core/transformer.cpp:126-141)
    assert abs(0.7978845608028654 - math.sqrt(2 / math.pi)) < 1e-15
    assert abs(0.70710678118654752440 - 1 / math.sqrt(2)) < 1e-15
    assert plain.ACTIVATIONS["gelu_new"] is plain.gelu_tanh and plain.ACTIVATIONS["gelu"] is plain.gelu_erf


@pytest.mark.parametrize("n_head,hd", [(1, 16), (4, 16), (3, 32)])
def test_attention_is_the_library_routine(n_head, hd):
    T, d = 23, n_head * hd
    q, k, v = (RNG.standard_normal((T, d)) for _ in range(3))
    scale = 0.37
    got = plain.causal_attention(q, k, v, n_head, scale)

    def heads(a):
        return torch.tensor(a).reshape(T, n_head, hd).transpose(0, 1)

    want = F.scaled_dot_product_attention(heads(q), heads(k), heads(v), is_causal=True, scale=scale)
    assert np.allclose(got, want.transpose(0, 1).reshape(T, d).numpy(), atol=1e-12)
    # without the mask, the last query is plain softmax attention over all keys
    full = F.scaled_dot_product_attention(heads(q)[:, -1:], heads(k), heads(v), scale=scale)
    assert np.allclose(got[-1], full.transpose(0, 1).reshape(d).numpy(), atol=1e-12)


def test_attention_invariants():
    T, n_head, hd = 40, 2, 16
    d = n_head * hd
    q, k, v = (RNG.standard_normal((T, d)) for _ in range(3))
    out = plain.causal_attention(q, k, v, n_head, 0.25)
    assert np.allclose(out[0], v[0])  # position 0 sees itself only
    k2, v2 = k.copy(), v.copy()
    k2[21:] += 5.0
    v2[21:] -= 3.0
    assert np.allclose(plain.causal_attention(q, k2, v2, n_head, 0.25)[:21], out[:21])  # causal
    # a peaked score picks one value row: own position included, nothing after it
    q3, k3 = np.zeros((T, d)), np.zeros((T, d))
    q3[30, :hd] = 1.0
    k3[30, :hd] = 200.0
    assert np.allclose(plain.causal_attention(q3, k3, v, n_head, 1.0)[30, :hd], v[30, :hd], atol=1e-9)
    # only distances count in a window: shifting the whole sequence changes nothing
    w = plain.causal_attention(q, k, v, n_head, 0.25, window=8)
    assert np.allclose(w[20], plain.causal_attention(q[5:], k[5:], v[5:], n_head, 0.25, window=8)[15])
    assert np.allclose(w[:8], out[:8]) and not np.allclose(w[20], out[20])
    # the scale multiplies the scores (not divides)
    assert not np.allclose(plain.causal_attention(q, k, v, n_head, 4.0), out)


def test_fused_qkv_is_three_projections_stacked():
    """tests/test_model.cpp:888-894, 930-936: the same draws as separate matrices, [q | k | v]."""
    d = 32
    h = RNG.standard_normal((7, d))
    wq, wk, wv = (RNG.standard_normal((d, d)) for _ in range(3))
    bq, bk, bv = (RNG.standard_normal(d) for _ in range(3))
    q, k, v = plain.qkv_projection(h, np.concatenate([wq, wk, wv], axis=1), np.concatenate([bq, bk, bv]))
    assert np.allclose(q, h @ wq + bq) and np.allclose(k, h @ wk + bk) and np.allclose(v, h @ wv + bv)


def test_attention_scale_options():
    base = {"n_embd": 64, "n_head": 4}
    assert plain.attention_scale(base, 0) == pytest.approx(0.25)
    assert plain.attention_scale(base, 5) == pytest.approx(0.25)
    inv = dict(base, scale_attn_by_inverse_layer_idx=True)
    assert plain.attention_scale(inv, 0) == pytest.approx(0.25)  # layer 0 is unaffected: 1 / (0 + 1)
    assert plain.attention_scale(inv, 2) == pytest.approx(0.25 / 3)
    assert plain.attention_scale(dict(base, scale_attn_weights=False), 3) == 1.0


def test_whole_model_structure(plain_models):
    """One layer by hand from library routines; causality; the tied head; both options of B."""
    config, tensors = plain_models["B"]
    ids = list(np.random.default_rng(5).integers(0, config["vocab_size"], 17))
    logits = plain.forward(config, tensors, ids)
    assert logits.shape == (17, config["vocab_size"])
    # by hand, with torch routines
    t = {k: torch.tensor(v) for k, v in tensors.items()}
    d, H = config["n_embd"], config["n_head"]
    x = t["wte.weight"][ids] + t["wpe.weight"][:17]
    for L in range(config["n_layer"]):
        p = f"h.{L}."
        h = F.layer_norm(x, (d,), t[p + "ln_1.weight"], t[p + "ln_1.bias"], config["layer_norm_epsilon"])
        q, k, v = (h @ t[p + "attn.c_attn.weight"] + t[p + "attn.c_attn.bias"]).split(d, dim=-1)
        sh = lambda a: a.reshape(17, H, d // H).transpose(0, 1)  # noqa: E731
        a = F.scaled_dot_product_attention(sh(q), sh(k), sh(v), is_causal=True, scale=1 / math.sqrt(d // H) / (L + 1))
        x = x + a.transpose(0, 1).reshape(17, d) @ t[p + "attn.c_proj.weight"] + t[p + "attn.c_proj.bias"]
        h = F.layer_norm(x, (d,), t[p + "ln_2.weight"], t[p + "ln_2.bias"], config["layer_norm_epsilon"])
        x = x + F.gelu(h @ t[p + "mlp.c_fc.weight"] + t[p + "mlp.c_fc.bias"]) @ t[p + "mlp.c_proj.weight"] + t[p + "mlp.c_proj.bias"]
    want = F.layer_norm(x, (d,), t["ln_f.weight"], t["ln_f.bias"], config["layer_norm_epsilon"]) @ t["wte.weight"].T
    assert np.allclose(logits, want.numpy(), atol=1e-10)
    # causality: changing a later token leaves earlier logits alone
    ids2 = list(ids)
    ids2[9] = (ids2[9] + 1) % config["vocab_size"]
    assert np.allclose(plain.forward(config, tensors, ids2)[:9], logits[:9])
    assert not np.allclose(plain.forward(config, tensors, ids2)[9:], logits[9:])
    # the tied head: changing wte moves embeddings and logits
    t2 = dict(tensors)
    t2["wte.weight"] = tensors["wte.weight"] * 1.5
    assert not np.allclose(plain.forward(config, t2, ids), logits)
    # the options of B are live: turning either off changes the logits
    for key, val in (("scale_attn_by_inverse_layer_idx", False), ("activation_function", "gelu_new"),
                     ("layer_norm_epsilon", 1e-2)):
        assert np.abs(plain.forward(dict(config, **{key: val}), tensors, ids) - logits).max() > 1e-6, key


def test_sampler_rules():
    logits = np.array([0.5, 2.0, 2.0, -1.0, 1.5], dtype=np.float32)
    assert np.argmax(plain.probabilities(logits, 0.0)) == 1  # ties go to the lowest id (sampling.cpp:12-14)
    p = plain.probabilities(logits, 1.0)
    want = np.exp(logits.astype(np.float64) - 2.0)
    assert np.allclose(p, want / want.sum(), atol=1e-7)
    pk = plain.probabilities(logits, 1.0, top_k=2)
    assert np.count_nonzero(pk) == 2 and pk[1] > 0 and pk[2] > 0 and abs(pk.sum() - 1) < 1e-12
    pp = plain.probabilities(logits, 1.0, top_p=0.5)  # shortest prefix whose share reaches 0.5
    assert np.count_nonzero(pp) == 2
    assert np.count_nonzero(plain.probabilities(logits, 1.0, top_p=0.2)) == 1
    cold = plain.probabilities(logits, 1e-3)
    assert cold[1] + cold[2] > 0.999999  # T -> 0 approaches greedy
    # the walk over ascending ids
    probs = np.array([0.1, 0.0, 0.6, 0.3])
    assert plain.sample(probs, 0.05) == 0 and plain.sample(probs, 0.1) == 2 and plain.sample(probs, 0.69999) == 2
    assert plain.sample(probs, 0.7) == 3 and plain.sample(probs, 0.999999) == 3
    u = [plain.uniform(4, i) for i in range(1000)]
    assert all(0.0 <= x < 1.0 for x in u) and 0.45 < np.mean(u) < 0.55 and len(set(u)) == 1000
    assert plain.uniform(4, 0) != plain.uniform(5, 0)


def test_rng_is_splitmix64s_output_function():
    """Pinned by the generator's published first outputs from state 0 (0xE220A8397B1DCDAF, then
    0x6E789E6AA1B965F4): (seed 0, index -1) makes the counter 0 and (seed 1, index -1) one
    increment, so that a wrong constant or shift in either copy of the formula fails."""
    from liyab_amd.sampling import uniform

    for fn in (plain.uniform, uniform):
        assert fn(0, -1) == (0xE220A8397B1DCDAF >> 11) / 2.0 ** 53
        assert fn(1, -1) == (0x6E789E6AA1B965F4 >> 11) / 2.0 ** 53
        assert fn(0, 0) != fn(0, -1) and 0.0 <= fn(7, 123) < 1.0


def test_rng_agrees_with_the_engine():
    from liyab_amd.sampling import uniform

    for seed in (1, 4, 2**63 + 5):
        for i in (0, 1, 31, 1000):
            assert uniform(seed, i) == plain.uniform(seed, i)


def test_bf16_rounding_matches_torch():
    a = np.random.default_rng(3).standard_normal(10000).astype(np.float32) * 3
    want = torch.tensor(a).to(torch.bfloat16).to(torch.float64).numpy()
    assert np.array_equal(plain.round_to_bf16(a), want)
