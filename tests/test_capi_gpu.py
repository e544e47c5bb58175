"""The engine as a C library (csrc/capi/liyab_engine_c.h): from a C program of its own, which
starts the interpreter inside its process, and through ctypes from this one (needs the GPU)."""

import ctypes
import os
import subprocess
import sysconfig

import pytest

import plain_gpt2 as plain
import trace_tools as tt
from conftest import CONFIGS, ROOT

pytestmark = pytest.mark.gpu


def _library():
    from liyab_amd.csrc import build

    path = os.path.join(build.PKG, "_lib", build.CAPI_LIB_NAME)
    if not os.path.isfile(path):
        path = build.build_engine_capi(quiet=True)
    return path


def test_a_c_program_generates_through_the_c_library(model_dirs, plain_models, tmp_path):
    from liyab_amd.csrc import build

    lib = _library()
    exe = str(tmp_path / "capi_driver")
    cc = build.cxx_path().replace("g++", "gcc") if os.path.exists(build.cxx_path().replace("g++", "gcc")) else build.cxx_path()
    libdir = os.path.dirname(lib)
    r = subprocess.run([cc, "-O1", "-Wall", "-I", build.CAPI_DIR, "-o", exe, os.path.join(ROOT, "tests", "capi_driver.c"),
                        f"-L{libdir}", "-lliyab_engine", f"-Wl,-rpath,{libdir}",
                        f"-Wl,-rpath,{sysconfig.get_config_var('LIBDIR')}"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    name = "A"
    config, tensors = plain_models[name]
    prompt = tt.random_tokens(31, 9, CONFIGS[name][0]["vocab_size"])
    p = subprocess.run([exe, model_dirs[name], "12", *map(str, prompt)], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, (p.stdout[-2000:], p.stderr[-4000:])
    lines = {l.split()[0] + (" " + l.split()[1] if l.startswith("bad") else ""): l for l in p.stdout.splitlines() if l.strip()}
    want = plain.generate_greedy(config, tensors, prompt, 12)
    assert lines["tokens"].split()[1:] == [str(t) for t in want]
    assert lines["stats"].split()[1:] == ["9", "12", "0"]
    assert lines["stopped"].split()[1:] == ["3", "1", *[str(t) for t in want[:3]]]
    assert lines["bad token:"].startswith("bad token: status 1:") and "outside" in lines["bad token:"]
    assert lines["bad folder:"].startswith("bad folder: status 2:") and "config.json" in lines["bad folder:"]


def test_the_c_library_through_ctypes(model_dirs, plain_models):
    class Config(ctypes.Structure):
        _fields_ = [("model_path", ctypes.c_char_p), ("dtype", ctypes.c_char_p)] + [
            (n, ctypes.c_int32) for n in ("context_length", "page_size", "num_pages", "max_sequences", "max_batched_tokens",
                                          "prefill_chunk", "batch_invariant")]

    class Params(ctypes.Structure):
        _fields_ = [("temperature", ctypes.c_float), ("top_k", ctypes.c_int32), ("top_p", ctypes.c_float),
                    ("seed", ctypes.c_uint64), ("max_tokens", ctypes.c_int32)]

    lib = ctypes.CDLL(_library())
    lib.liyab_engine_last_error.restype = ctypes.c_char_p
    cfg, sp = Config(), Params()
    lib.liyab_engine_config_default(ctypes.byref(cfg))
    lib.liyab_sampling_params_default(ctypes.byref(sp))
    assert (cfg.page_size, cfg.prefill_chunk, cfg.dtype) == (16, 256, b"bfloat16")
    assert (round(sp.temperature, 3), sp.top_k, round(sp.top_p, 3), sp.seed, sp.max_tokens) == (0.8, 40, 0.95, 0, 256)
    name = "B"
    config, tensors = plain_models[name]
    cfg.model_path, cfg.dtype, cfg.context_length = model_dirs[name].encode(), b"float32", 128
    engine = ctypes.c_void_p()
    assert lib.liyab_engine_create(ctypes.byref(cfg), ctypes.byref(engine)) == 0, lib.liyab_engine_last_error()
    prompt = tt.random_tokens(32, 20, CONFIGS[name][0]["vocab_size"])
    ids = (ctypes.c_int32 * len(prompt))(*prompt)
    out = (ctypes.c_int32 * 64)()
    n_out = ctypes.c_size_t()
    sp.temperature, sp.max_tokens = 0.0, 10
    seen = []
    callback = ctypes.CFUNCTYPE(ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p)(lambda t, u: seen.append(t) or 1)
    rc = lib.liyab_engine_generate_tokens(engine, ids, len(prompt), ctypes.byref(sp), callback, None, out, 64,
                                          ctypes.byref(n_out), None)
    assert rc == 0, lib.liyab_engine_last_error()
    want = plain.generate_greedy(config, tensors, prompt, 10)
    assert list(out[:n_out.value]) == want == seen
    # a prompt longer than the context that was asked for
    long_ids = (ctypes.c_int32 * 200)(*([1] * 200))
    rc = lib.liyab_engine_generate_tokens(engine, long_ids, 200, ctypes.byref(sp), None, None, out, 64, ctypes.byref(n_out), None)
    assert rc == 1 and b"context" in lib.liyab_engine_last_error()
    lib.liyab_engine_destroy(engine)
