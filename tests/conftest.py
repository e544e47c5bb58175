"""Shared fixtures: two tiny GPT-2 configurations that differ in every size and
option, model folders with random weights, and the GPU marker."""

import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

# A: 2 layers, width 64, 4 heads of 16, 4x feed-forward, tanh GELU, eps 1e-5
CONFIG_A = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2",
    "n_layer": 2, "n_embd": 64, "n_head": 4, "n_inner": None, "vocab_size": 512, "n_positions": 128,
    "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new", "scale_attn_by_inverse_layer_idx": False,
    "scale_attn_weights": True, "tie_word_embeddings": True,
}
# B: 3 layers, width 96, 3 heads of 32, feed-forward 320 (not 4x, no power of two), vocabulary 1000,
# erf GELU, eps 1e-6, attention scaled by 1 / (layer + 1) too
CONFIG_B = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2",
    "n_layer": 3, "n_embd": 96, "n_head": 3, "n_inner": 320, "vocab_size": 1000, "n_positions": 256,
    "layer_norm_epsilon": 1e-6, "activation_function": "gelu", "scale_attn_by_inverse_layer_idx": True,
    "scale_attn_weights": True, "tie_word_embeddings": True,
}
# C: odd sizes for the kernels: width 144 = 3 heads of 48, vocabulary 777, one layer
CONFIG_C = {
    "architectures": ["GPT2LMHeadModel"], "model_type": "gpt2",
    "n_layer": 1, "n_embd": 144, "n_head": 3, "n_inner": 200, "vocab_size": 777, "n_positions": 640,
    "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new", "scale_attn_by_inverse_layer_idx": False,
    "scale_attn_weights": True, "tie_word_embeddings": True,
}
CONFIGS = {"A": (CONFIG_A, 0), "B": (CONFIG_B, 2), "C": (CONFIG_C, 5)}

# Tolerances, relative to the largest |logit| of the compared row; fixed, never widened to pass.
# A test session prints the largest error each family of checks saw (pytest_terminal_summary below).
# float32: the engine's families show 0.5e-6 to 3.2e-6 (the largest at GPT-2 XL's layer sizes).
# bfloat16, GPT-2 models with the benchmark's weight distributions: 2.6e-3 to 6.4e-3 (the largest at
# XL's layer sizes again); the tolerance is twice that largest. It was 2e-2 before the errors were on record.
TOL = {"float32": 1e-5, "bfloat16": 1.3e-2}
# The toy models of test_parts_gpu.py draw weights five to ten times as large and run torch arithmetic
# of their own between the framework's kernels (values rounded to bfloat16 twice): 7.8e-3 to 1.27e-2.
TOL_TOY = {"float32": 1e-5, "bfloat16": 2e-2}


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_terminal_summary(terminalreporter):
    """The largest relative error each family of logit checks saw, beside its tolerance."""
    import trace_tools

    if trace_tools.WORST:
        terminalreporter.write_line("largest relative error of the engine's logits against the plain implementation:")
        for (family, tol), worst in sorted(trace_tools.WORST.items(), key=lambda kv: (kv[0][1], kv[0][0])):
            terminalreporter.write_line(f"  {family:<24} tolerance {tol:.0e}  worst {worst:.3e}  ({worst / tol:.2f} of it)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """{name: folder} with float32 weights for A, B, C (made once a session, in a temporary folder)."""
    from liyab_amd.weights import write_random_model

    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        d = tmp_path_factory.mktemp(f"model_{name}")
        write_random_model(str(d), dict(cfg), seed)
        out[name] = str(d)
    return out


@pytest.fixture(scope="session")
def plain_models(model_dirs):
    """{name: (config, float64 tensors)} read by the plain implementation."""
    import plain_gpt2 as plain

    return {name: plain.read_model(d) for name, d in model_dirs.items()}
