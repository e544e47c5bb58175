"""Each part alone against its plain formula, and the generality of the layer plan: a toy
mixer with state of its own, a feed-forward that routes and a position encoding without a
table, defined here, are registered, built and stepped without touching the framework's files; a layer
reads another layer's cache; the run order names a layer twice; a norm of another kind and blocks arranged
otherwise (parallel, post-norm) (needs the GPU)."""

import math
import os

import numpy as np
import pytest
import torch

import plain_gpt2 as plain
import trace_tools as tt
from conftest import TOL, TOL_TOY

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def T(name, layout="out_in", required=True):
    from liyab_amd.config import TensorSource

    return TensorSource(name, layout, required)


def norm_spec(prefix, d, eps):
    from liyab_amd.config import NormSpec

    return NormSpec("layernorm", d, eps, {"weight": T(prefix + ".w"), "bias": T(prefix + ".b")})


def attention_spec(prefix, d, H, Hkv, hd, scale, window=0):
    from liyab_amd.config import AttentionSpec

    return AttentionSpec("attention", d, H, Hkv, hd, scale, window,
                         {"qkv_weight": T(prefix + ".qkv.w"), "qkv_bias": T(prefix + ".qkv.b"),
                          "out_weight": T(prefix + ".out.w"), "out_bias": T(prefix + ".out.b")})


def ffn_spec(prefix, d, F, act):
    from liyab_amd.config import DenseFFNSpec

    return DenseFFNSpec("dense_ffn", d, F, act, {"up_weight": T(prefix + ".up.w"), "up_bias": T(prefix + ".up.b"),
                                                 "down_weight": T(prefix + ".down.w"), "down_bias": T(prefix + ".down.b")})


def make_plan(d, V, P, layers, order, eps=1e-5):
    from liyab_amd.config import HeadSpec, ModelPlan, PositionSpec, TokenEmbeddingSpec

    return ModelPlan(architecture="toy", width=d, vocab_size=V, max_positions=P,
                     embedding=TokenEmbeddingSpec("token_embedding", V, d, 1.0, {"table": T("emb")}),
                     residual_position=PositionSpec("learned_positions", "residual", P, d, {"table": T("pos")}),
                     layers=layers, order=order, final_norm=norm_spec("nf", d, eps),
                     head=HeadSpec("lm_head", d, V, 1.0, {"weight": T("emb")}))


def rand(rng, *shape, scale=1.0, mean=0.0):
    return torch.from_numpy((rng.standard_normal(shape) * scale + mean).astype(np.float32))


def norm_tensors(rng, prefix, d):
    return {prefix + ".w": rand(rng, d, scale=0.1, mean=1.0), prefix + ".b": rand(rng, d, scale=0.1)}


def attention_tensors(rng, prefix, d, H, Hkv, hd):
    n = (H + 2 * Hkv) * hd
    return {prefix + ".qkv.w": rand(rng, n, d, scale=0.15), prefix + ".qkv.b": rand(rng, n, scale=0.1),
            prefix + ".out.w": rand(rng, d, H * hd, scale=0.1), prefix + ".out.b": rand(rng, d, scale=0.1)}


def ffn_tensors(rng, prefix, d, F):
    return {prefix + ".up.w": rand(rng, F, d, scale=0.15), prefix + ".up.b": rand(rng, F, scale=0.1),
            prefix + ".down.w": rand(rng, d, F, scale=0.1), prefix + ".down.b": rand(rng, d, scale=0.1)}


def f64(t):
    return t.double().numpy()


# ---------------------------------------------------------------------------
# plain formulas for the toy models (whole sequences, float64)
# ---------------------------------------------------------------------------
def plain_attention(h, tw, prefix, H, Hkv, hd, scale, window=0, kv_from=None, rotate=None):
    """QKV with [out, in] weights, grouped heads, optional window; `kv_from` = (k, v) of another
    layer; `rotate(x, heads)` acts on queries and keys before any score."""
    qkv = h @ f64(tw[prefix + ".qkv.w"]).T + f64(tw[prefix + ".qkv.b"])
    q, k, v = qkv[:, :H * hd], qkv[:, H * hd:(H + Hkv) * hd], qkv[:, (H + Hkv) * hd:]
    if rotate is not None:
        q, k = rotate(q, H), rotate(k, Hkv)
    if kv_from is not None:
        k, v = kv_from
    rep = H // Hkv
    # query head hh reads key/value head hh // rep
    kk = np.concatenate([k[:, (hh // rep) * hd:(hh // rep + 1) * hd] for hh in range(H)], axis=1)
    vv = np.concatenate([v[:, (hh // rep) * hd:(hh // rep + 1) * hd] for hh in range(H)], axis=1)
    att = plain.causal_attention(q, kk, vv, H, scale, window)
    return att @ f64(tw[prefix + ".out.w"]).T + f64(tw[prefix + ".out.b"]), (k, v)


def plain_ffn(h, tw, prefix, act):
    fn = plain.gelu_tanh if act == "gelu_tanh" else plain.gelu_erf
    return fn(h @ f64(tw[prefix + ".up.w"]).T + f64(tw[prefix + ".up.b"])) @ f64(tw[prefix + ".down.w"]).T + f64(tw[prefix + ".down.b"])


def plain_norm(x, tw, prefix, eps):
    return plain.layer_norm(x, f64(tw[prefix + ".w"]), f64(tw[prefix + ".b"]), eps)


# ---------------------------------------------------------------------------
# each part alone
# ---------------------------------------------------------------------------
class _Parts:
    """A one-layer engine whose step context and cache the part tests borrow."""

    def __init__(self, dtype, d=80, H=5, Hkv=5, hd=16, F=136, V=300, P=200, window=0, eps=1e-4, act="gelu_erf"):
        from liyab_amd.config import LayerSpec, OrderEntry
        from liyab_amd.engine import EngineCore

        rng = np.random.default_rng(7)
        self.d, self.H, self.Hkv, self.hd, self.F, self.V, self.eps, self.act = d, H, Hkv, hd, F, V, eps, act
        self.scale = 0.9 / math.sqrt(hd)
        layer = LayerSpec(attention_spec("a", d, H, Hkv, hd, self.scale, window), ffn_spec("f", d, F, act),
                          norm_spec("n1", d, eps), norm_spec("n2", d, eps))
        self.tw = {"emb": rand(rng, V, d, scale=0.5), "pos": rand(rng, P, d, scale=0.3), **norm_tensors(rng, "nf", d),
                   **norm_tensors(rng, "n1", d), **norm_tensors(rng, "n2", d), **attention_tensors(rng, "a", d, H, Hkv, hd),
                   **ffn_tensors(rng, "f", d, F)}
        if dtype == "bfloat16":  # the bfloat16 path holds matrices in bfloat16: compare against those values
            self.tw = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v) for k, v in self.tw.items()}
        self.core = EngineCore.from_plan(make_plan(d, V, P, [layer], [OrderEntry(0)], eps), self.tw, dtype=dtype,
                                         page_size=8, num_pages=64, max_requests=4, use_graphs=False)
        self.block = self.core.model.blocks[0]


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def parts(request):
    return _Parts(request.param), request.param


def test_embedding_and_positions_alone(parts):
    from liyab_amd.engine import StepItem

    p, dtype = parts
    core = p.core
    core.open("e")
    ids = [5, 299, 0, 17, 5]
    core.step([StepItem("e", [1, 2, 3], [])])  # so that the next tokens sit at positions 3..7
    ctx, lengths = core.step_fn.prepare([StepItem("e", ids, [])])
    x = torch.zeros(5, p.d, device=DEV)
    core.model.embedding.forward(ctx, x)
    assert torch.equal(x.cpu(), core.model.embedding.table.float().cpu()[ids])
    core.model.residual_position.add(ctx, x)
    want = f64(p.tw["emb"])[ids] + f64(p.tw["pos"])[3:8]
    assert tt.rel_err(x.cpu().numpy(), want) < 1e-6
    x2 = torch.zeros(5, p.d, device=DEV)
    core.model.embedding.forward(ctx, x2, position_table=core.model.residual_position.fused_table())
    assert torch.equal(x2, x)
    core.step_fn.commit([StepItem("e", ids, [])], lengths)
    core.close("e")


def test_norm_alone(parts):
    from liyab_amd.engine import StepItem

    p, dtype = parts
    core = p.core
    core.open("n")
    ctx, _ = core.step_fn.prepare([StepItem("n", [1] * 9, [2, 7])])
    x = rand(np.random.default_rng(1), 9, p.d, scale=2.0, mean=0.7).to(DEV)
    tol = 1e-5 if dtype == "float32" else 6e-3
    got = p.block.norm_mixer.forward(x, ctx)
    assert tt.rel_err(got.float().cpu().numpy(), plain_norm(f64(x.cpu()), p.tw, "n1", p.eps)) < tol
    got = core.model.final_norm.forward(x, ctx, rows=ctx.logit_rows, n_rows=2, name="t")
    assert tt.rel_err(got.float().cpu().numpy(), plain_norm(f64(x.cpu())[[2, 7]], p.tw, "nf", p.eps)) < tol
    pending = p.block.norm_ffn.lazy(x, ctx)
    assert pending.shape == (9, p.d)
    assert tt.rel_err(pending.tensor().float().cpu().numpy(), plain_norm(f64(x.cpu()), p.tw, "n2", p.eps)) < tol
    core.close("n")


@pytest.mark.parametrize("lazy", [False, True, "unfolded"])
def test_feed_forward_alone(parts, lazy, monkeypatch):
    from liyab_amd.engine import StepItem
    from liyab_amd.parts import linear

    if lazy == "unfolded":  # without the product kernel that applies a pending norm itself
        monkeypatch.setattr(linear, "FOLD_NORM", False)
    p, dtype = parts
    core = p.core
    core.open("f")
    ctx, _ = core.step_fn.prepare([StepItem("f", [1] * 11, [])])
    rng = np.random.default_rng(2)
    x = rand(rng, 11, p.d, scale=1.5).to(DEV)
    residual = rand(rng, 11, p.d).to(DEV)
    want = f64(residual.cpu()) + plain_ffn(plain_norm(f64(x.cpu()), p.tw, "n2", p.eps), p.tw, "f", p.act)
    h = p.block.norm_ffn.lazy(x, ctx) if lazy else p.block.norm_ffn.forward(x, ctx)
    p.block.ffn.forward(h, ctx, residual)
    assert tt.rel_err(residual.cpu().numpy(), want) < (1e-5 if dtype == "float32" else 1e-2)
    core.close("f")


@pytest.mark.parametrize("reader", ["norm", "gathering norm", "settle", "product"])
@pytest.mark.parametrize("split_before", [False, True])
def test_feed_forward_deferred(parts, reader, split_before, monkeypatch):
    """The feed-forward's second product cut over its inner dimension: the stream comes back
    split into planes (the stream's own tensor untouched), and the next reader adds them up: a
    norm as it loads its rows, a norm over gathered rows, a product with the norm folded in, or
    a pass of its own into the stream's tensor. The stream may have been split already."""
    from liyab_amd.engine import StepItem
    from liyab_amd.kernels import ops
    from liyab_amd.parts.base import SplitStream
    from liyab_amd.parts.linear import linear

    p, dtype = parts
    if dtype != "bfloat16":
        pytest.skip("only the bfloat16 products are cut over K")
    monkeypatch.setattr(ops, "k_parts", lambda M, N, K: 3)  # the sizes here would not be cut
    core = p.core
    core.open("f")
    ctx, _ = core.step_fn.prepare([StepItem("f", [1] * 11, [])])
    rng = np.random.default_rng(2)
    x = rand(rng, 11, p.d, scale=1.5).to(DEV)
    residual = rand(rng, 11, p.d).to(DEV)
    want = f64(residual.cpu()) + plain_ffn(plain_norm(f64(x.cpu()), p.tw, "n2", p.eps), p.tw, "f", p.act)
    stream = residual
    if split_before:  # the stream arrives as two planes that add up to `residual`; its tensor is stale
        half = rand(rng, 11, p.d).to(DEV)
        stream = SplitStream(torch.stack([residual - half, half]), torch.full_like(residual, float("nan")))
    home = stream.home if split_before else residual
    before = home.clone()
    split = p.block.ffn.forward(p.block.norm_ffn.forward(x, ctx), ctx, stream, defer=True)
    assert isinstance(split, SplitStream) and split.planes.shape == (3, 11, p.d) and split.home is home
    assert split_before or torch.equal(home, before)  # untouched (NaN never equals itself)
    norm = p.block.norm_mixer
    assert norm.takes_planes(split.planes)
    if reader == "norm":
        got = norm.forward(split.planes, ctx).float().cpu().numpy()
        assert tt.rel_err(got, plain_norm(want, p.tw, "n1", p.eps)) < 1e-2
    elif reader == "gathering norm":
        rows = torch.tensor([7, 0, 7, 10], dtype=torch.int32, device=DEV)
        got = norm.forward(split.planes, ctx, rows=rows).float().cpu().numpy()
        assert tt.rel_err(got, plain_norm(want[[7, 0, 7, 10]], p.tw, "n1", p.eps)) < 1e-2
    elif reader == "product":
        w = rand(rng, 24, p.d).to(DEV).to(torch.bfloat16)
        out = torch.empty(11, 24, dtype=torch.bfloat16, device=DEV)
        linear(norm.lazy(split.planes, ctx), w, None, out=out)
        ref = plain_norm(want, p.tw, "n1", p.eps) @ f64(w.float().cpu()).T
        assert tt.rel_err(out.float().cpu().numpy(), ref) < 2e-2
    assert split.settle() is home
    assert tt.rel_err(home.cpu().numpy(), want) < 1e-2
    core.close("f")


@pytest.mark.parametrize("split_before", [False, True])
def test_product_of_a_tile_of_rows_deferred_through_the_tiled_kernel(parts, split_before, monkeypatch):
    """A product of 33 to 64 rows that is added to the stream, cut over K through the tiled
    kernel (forced here: the rule takes only long inner dimensions): the stream comes back split,
    its planes adding up to stream + a . W^T + bias, whether it was whole or split before."""
    from liyab_amd.engine import StepItem
    from liyab_amd.kernels import ops
    from liyab_amd.parts.base import SplitStream
    from liyab_amd.parts.linear import linear_deferred

    p, dtype = parts
    if dtype != "bfloat16":
        pytest.skip("only the bfloat16 products are cut over K")
    monkeypatch.setattr(ops, "tiled_k_parts", lambda M, N, K: 3)
    core = p.core
    core.open("f")
    ctx, _ = core.step_fn.prepare([StepItem("f", [1] * 40, [])])
    rng = np.random.default_rng(5)
    a = rand(rng, 40, 320).to(DEV).to(torch.bfloat16)
    w = rand(rng, 72, 320, scale=0.1).to(DEV).to(torch.bfloat16)
    bias = rand(rng, 72).to(DEV)
    residual = rand(rng, 40, 72).to(DEV)
    stream = residual
    if split_before:
        half = rand(rng, 40, 72).to(DEV)
        stream = SplitStream(torch.stack([residual - half, half]), torch.full_like(residual, float("nan")))
    assert ops.k_parts(40, 72, 320) == 1
    split = linear_deferred(a, w, bias, ctx, "tiled_parts_test", stream)
    assert isinstance(split, SplitStream) and split.planes.shape == (3, 40, 72)
    want = f64(residual.cpu()) + f64(a.float().cpu()) @ f64(w.float().cpu()).T + f64(bias.cpu())
    assert tt.rel_err(split.settle().cpu().numpy(), want) < 1e-5
    core.close("f")


@pytest.mark.parametrize("rows,n_planes", [(40, 3), (64, 1), (7, 2)])
def test_product_that_is_not_cut_takes_a_split_stream(parts, rows, n_planes, monkeypatch):
    """A product of few rows that is not worth cutting over K, added to a stream that arrives
    split: the streaming kernel adds the stream's planes in its epilogue and leaves one plane
    (the stream's own tensor stays stale, no pass to settle it first); a whole stream is left to
    the caller as before."""
    from liyab_amd.engine import StepItem
    from liyab_amd.kernels import ops
    from liyab_amd.parts.base import SplitStream
    from liyab_amd.parts.linear import linear_deferred

    p, dtype = parts
    if dtype != "bfloat16":
        pytest.skip("only the bfloat16 products take planes")
    monkeypatch.setattr(ops, "k_parts", lambda M, N, K: 1)
    core = p.core
    core.open("f")
    ctx, _ = core.step_fn.prepare([StepItem("f", [1] * rows, [])])
    rng = np.random.default_rng(6)
    a = rand(rng, rows, 200).to(DEV).to(torch.bfloat16)
    w = rand(rng, 88, 200, scale=0.1).to(DEV).to(torch.bfloat16)
    bias = rand(rng, 88).to(DEV)
    residual = rand(rng, rows, 88).to(DEV)
    assert linear_deferred(a, w, bias, ctx, "uncut_test", residual) is None  # a whole stream: the caller's plain product
    planes = torch.stack([rand(rng, rows, 88).to(DEV) for _ in range(n_planes)])
    planes[0] += residual - planes.sum(dim=0)
    home = torch.full_like(residual, float("nan"))
    split = linear_deferred(a, w, bias, ctx, "uncut_test", SplitStream(planes, home))
    assert isinstance(split, SplitStream) and split.planes.shape == (1, rows, 88) and split.home is home
    assert torch.isnan(home).all()
    want = f64(residual.cpu()) + f64(a.float().cpu()) @ f64(w.float().cpu()).T + f64(bias.cpu())
    assert tt.rel_err(split.planes[0].cpu().numpy(), want) < 1e-5
    assert tt.rel_err(split.settle().cpu().numpy(), want) < 1e-5
    core.close("f")


@pytest.mark.parametrize("geometry", [dict(H=5, Hkv=5, hd=16), dict(H=6, Hkv=2, hd=32, d=96), dict(H=3, Hkv=1, hd=48, d=64, window=13)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_mixer_alone(dtype, geometry):
    """The mixer over its own cache: a whole portion, then more portions and single tokens,
    against plain attention over the whole sequence; grouped heads and a window too."""
    from liyab_amd.engine import StepItem

    p = _Parts(dtype, **geometry)
    core, att = p.core, p.block.mixer
    rng = np.random.default_rng(3)
    n = 60
    x = rand(rng, n, p.d, scale=1.2)
    want, _ = plain_attention(plain_norm(f64(x), p.tw, "n1", p.eps), p.tw, "a", p.H, p.Hkv, p.hd, p.scale,
                              window=geometry.get("window", 0))
    core.open("m")
    done = 0
    for take in (25, 1, 9, 1, 1, 23):
        item = StepItem("m", [1] * take, [])
        ctx, lengths = core.step_fn.prepare([item])
        xs = x[done:done + take].to(DEV)
        residual = torch.zeros(take, p.d, device=DEV)
        att.forward(p.block.norm_mixer.forward(xs, ctx), ctx, core.storage.layer(0), None, residual)
        core.step_fn.commit([item], lengths)
        err = tt.rel_err(residual.cpu().numpy(), want[done:done + take])
        assert err < (1e-5 if dtype == "float32" else 1e-2), (take, done, err)
        done += take
    core.close("m")
    core.manager.check()


def test_block_and_head_alone(parts):
    from liyab_amd.engine import StepItem

    p, dtype = parts
    core = p.core
    core.open("b")
    rng = np.random.default_rng(4)
    n = 21
    x0 = rand(rng, n, p.d, scale=1.1)
    item = StepItem("b", [1] * n, [0, n - 1])
    ctx, lengths = core.step_fn.prepare([item])
    x = x0.clone().to(DEV)
    p.block.forward(x, ctx, core.storage.layer(0), None)
    core.step_fn.commit([item], lengths)
    a, _ = plain_attention(plain_norm(f64(x0), p.tw, "n1", p.eps), p.tw, "a", p.H, p.Hkv, p.hd, p.scale)
    want = f64(x0) + a
    want = want + plain_ffn(plain_norm(want, p.tw, "n2", p.eps), p.tw, "f", p.act)
    assert tt.rel_err(x.cpu().numpy(), want) < (1e-5 if dtype == "float32" else 1e-2)
    h = core.model.final_norm.lazy(x, ctx, rows=ctx.logit_rows, n_rows=2, name="head_in")
    logits = core.model.head.forward(h, ctx)
    want_logits = plain_norm(want[[0, n - 1]], p.tw, "nf", p.eps) @ f64(p.tw["emb"]).T
    assert logits.dtype == torch.float32 and logits.shape == (2, p.V)
    assert tt.rel_err(logits.cpu().numpy(), want_logits) < (1e-5 if dtype == "float32" else 1.5e-2)
    core.close("b")


# ---------------------------------------------------------------------------
# a toy architecture: a mixer with state of its own, shared caches, a layer named twice
# ---------------------------------------------------------------------------
class DecaySpec:
    """Spec of the toy mixer: any object with a `kind` can stand in a LayerSpec."""

    kind = "toy_decay"

    def __init__(self, width, decay, prefix):
        self.width, self.decay, self.prefix = width, decay, prefix


class DecayMixer:
    """s_t = decay * s_{t-1} + h_t per request (state of fixed size, no keys), out = s_t . W^T.
    It keeps its state in the slot the cache manager gives its request, carries it across
    portions and steps, and uses torch for its arithmetic: it is a test's toy, not a kernel."""

    def __init__(self, spec, store, dtype):
        from liyab_amd.config import TensorSource

        self.width, self.decay, self.dtype = spec.width, spec.decay, dtype
        self.weight = store.fetch(TensorSource(spec.prefix + ".w"), (spec.width, spec.width), "matrix")

    def cache_spec(self):
        return None

    def state_spec(self):
        from liyab_amd.cache import StateSpec

        return StateSpec((self.width,), "float32")

    def forward(self, h, ctx, cache, state, residual, writes_cache=True):
        from liyab_amd.parts import as_tensor

        h = as_tensor(h).float()
        slots = ctx.state_slots.tolist()
        out = torch.empty_like(h)
        for i, (a, n) in enumerate(zip(ctx.host.starts, ctx.host.q_lens)):
            s = state[slots[i]]
            for t in range(a, a + n):  # in token order within the request's portion
                s = self.decay * s + h[t]
                out[t] = s
            state[slots[i]] = s
        residual += out @ self.weight.float().t()


def toy_model(dtype="float32"):
    """Layers: 0 = decay mixer + erf FFN, 1 = attention (5 heads of 16) + tanh FFN, 2 = windowed
    grouped attention (4 query heads on 2 key/value heads of 32, window 24) + tanh FFN, 3 =
    attention without a feed-forward that reads layer 1's cache. Run order 0, 1, 2, 3, 1
    (layer 1 a second time, reading its cache without writing)."""
    from liyab_amd.config import LayerSpec, OrderEntry
    from liyab_amd.parts import register_mixer

    register_mixer("toy_decay", DecayMixer)
    d, V, P, eps = 80, 211, 160, 1e-5
    rng = np.random.default_rng(11)
    s1 = 1 / math.sqrt(16)
    layers = [
        LayerSpec(DecaySpec(d, 0.8, "m0"), ffn_spec("f0", d, 100, "gelu_erf"), norm_spec("n0a", d, eps), norm_spec("n0b", d, eps)),
        LayerSpec(attention_spec("a1", d, 5, 5, 16, s1), ffn_spec("f1", d, 160, "gelu_tanh"), norm_spec("n1a", d, eps), norm_spec("n1b", d, eps)),
        LayerSpec(attention_spec("a2", d, 4, 2, 32, 0.2, window=24), ffn_spec("f2", d, 64, "gelu_tanh"), norm_spec("n2a", d, eps), norm_spec("n2b", d, eps)),
        LayerSpec(attention_spec("a3", d, 5, 5, 16, s1 / 2), None, norm_spec("n3a", d, eps), None),
    ]
    order = [OrderEntry(0), OrderEntry(1), OrderEntry(2), OrderEntry(3, cache_of=1, writes_cache=False),
             OrderEntry(1, writes_cache=False)]
    tw = {"emb": rand(rng, V, d, scale=0.5), "pos": rand(rng, P, d, scale=0.3), **norm_tensors(rng, "nf", d),
          "m0.w": rand(rng, d, d, scale=0.05)}
    for i, (H, Hkv, hd, F) in enumerate([(0, 0, 0, 100), (5, 5, 16, 160), (4, 2, 32, 64), (5, 5, 16, 0)]):
        tw.update(norm_tensors(rng, f"n{i}a", d))
        if F:
            tw.update(norm_tensors(rng, f"n{i}b", d))
            tw.update(ffn_tensors(rng, f"f{i}", d, F))
        if H:
            tw.update(attention_tensors(rng, f"a{i}", d, H, Hkv, hd))
    if dtype == "bfloat16":
        tw = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v) for k, v in tw.items()}
    return make_plan(d, V, P, layers, order, eps), tw, dict(d=d, V=V, P=P, eps=eps, s1=s1)


def toy_plain(tw, info, ids):
    """The toy model over a whole sequence, float64."""
    eps, s1 = info["eps"], info["s1"]
    x = f64(tw["emb"])[ids] + f64(tw["pos"])[:len(ids)]
    # layer 0: the decay mixer
    h = plain_norm(x, tw, "n0a", eps)
    s = np.zeros(info["d"])
    out = np.zeros_like(h)
    for t in range(len(ids)):
        s = 0.8 * s + h[t]
        out[t] = s
    x = x + out @ f64(tw["m0.w"]).T
    x = x + plain_ffn(plain_norm(x, tw, "n0b", eps), tw, "f0", "gelu_erf")
    # layer 1
    a, kv1 = plain_attention(plain_norm(x, tw, "n1a", eps), tw, "a1", 5, 5, 16, s1)
    x = x + a
    x = x + plain_ffn(plain_norm(x, tw, "n1b", eps), tw, "f1", "gelu_tanh")
    # layer 2: windowed, grouped
    a, _ = plain_attention(plain_norm(x, tw, "n2a", eps), tw, "a2", 4, 2, 32, 0.2, window=24)
    x = x + a
    x = x + plain_ffn(plain_norm(x, tw, "n2b", eps), tw, "f2", "gelu_tanh")
    # layer 3 reads layer 1's keys and values; no feed-forward
    a, _ = plain_attention(plain_norm(x, tw, "n3a", eps), tw, "a3", 5, 5, 16, s1 / 2, kv_from=kv1)
    x = x + a
    # layer 1 again, on its cache as its first run left it
    a, _ = plain_attention(plain_norm(x, tw, "n1a", eps), tw, "a1", 5, 5, 16, s1, kv_from=kv1)
    x = x + a
    x = x + plain_ffn(plain_norm(x, tw, "n1b", eps), tw, "f1", "gelu_tanh")
    return plain_norm(x, tw, "nf", eps) @ f64(tw["emb"]).T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_a_stateful_mixer(dtype):
    from liyab_amd.engine import EngineCore

    plan, tw, info = toy_model(dtype)
    reqs = {f"t{i}": tt.random_tokens(90 + i, n, info["V"]) for i, n in enumerate([37, 90, 5, 128, 61])}
    ref = {rid: toy_plain(tw, info, toks) for rid, toks in reqs.items()}
    tol = TOL_TOY[dtype]
    for name, steps in (("whole", tt.schedule_whole(reqs)), ("portions", tt.schedule_portions(reqs, (5, 2, 17, 3, 48))),
                        ("mixed", tt.schedule_mixed(reqs, seed=3))):
        core = EngineCore.from_plan(plan, tw, dtype=dtype, page_size=8, max_tokens=tt.max_live_tokens(steps), max_requests=4,
                                    use_graphs=False)  # the toy mixer reads its slots on the host: no capture
        groups = core.manager.groups
        assert len(groups) == 2 and sorted(g.spec.window for g in groups) == [0, 24]
        assert [g.layers for g in groups if g.spec.window == 0] == [[1]]  # layer 3 owns no cache: it reads layer 1's
        assert set(core.storage.states) == {0}  # only the decay mixer keeps state
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, ref, tol, f"toy {name} {dtype}")
        core.manager.check()
        assert all(core.manager.pages_in_use(g.index) == 0 for g in groups)


# ---------------------------------------------------------------------------
# more toy parts: a feed-forward with routing and a position encoding without a table
# ---------------------------------------------------------------------------
class RoutedSpec:
    kind = "toy_routed"

    def __init__(self, width, inner, n_experts, top, prefix):
        self.width, self.inner, self.n_experts, self.top, self.prefix = width, inner, n_experts, top, prefix


class RoutedFFN:
    """Router logits h . Wr^T in float32; the `top` largest experts of a token (ties to the lower
    index), a softmax over those; each expert an ungated tanh-GELU feed-forward without biases.
    A test's toy in torch: the framework's files know nothing of routing."""

    def __init__(self, spec, store, dtype):
        from liyab_amd.config import TensorSource

        self.top, self.dtype = spec.top, dtype
        self.router = store.fetch(TensorSource(spec.prefix + ".router"), (spec.n_experts, spec.width), "matrix")
        self.up = [store.fetch(TensorSource(f"{spec.prefix}.{e}.up"), (spec.inner, spec.width), "matrix") for e in range(spec.n_experts)]
        self.down = [store.fetch(TensorSource(f"{spec.prefix}.{e}.down"), (spec.width, spec.inner), "matrix") for e in range(spec.n_experts)]

    def forward(self, h, ctx, residual):
        from liyab_amd.parts import as_tensor

        h = as_tensor(h).float()
        logits = h @ self.router.float().t()
        top = torch.topk(logits, self.top, dim=1, sorted=True)  # equal logits do not occur with these weights
        gates = torch.softmax(top.values, dim=1)
        out = torch.zeros_like(h)
        for e in range(len(self.up)):
            rows, which = (top.indices == e).nonzero(as_tuple=True)
            if rows.numel():
                m = torch.nn.functional.gelu(h[rows] @ self.up[e].float().t(), approximate="tanh") @ self.down[e].float().t()
                out.index_add_(0, rows, m * gates[rows, which].unsqueeze(1))
        residual += out


class SinusoidSpec:
    kind = "toy_sinusoid"

    def __init__(self, width, base):
        self.width, self.base = width, base


class SinusoidPositions:
    """x[t, 2i] += sin(pos_t / base^(2i / d)), x[t, 2i + 1] += cos(the same): computed from the
    positions of the step's tokens, no table and no limit to the context of its own."""

    where = "residual"

    def __init__(self, spec, store, dtype):
        self.width, self.base = spec.width, spec.base

    def fused_table(self):
        return None  # nothing the embedding kernel could add in its pass

    def add(self, ctx, x):
        i = torch.arange(0, self.width, 2, device=x.device, dtype=torch.float64)
        angle = ctx.positions.double().unsqueeze(1) / self.base ** (i / self.width)
        x[:, 0::2] += angle.sin().to(x.dtype)
        x[:, 1::2] += angle.cos().to(x.dtype)


def routed_model(dtype):
    """Layer 0: attention (3 heads of 16) + routed feed-forward (top 2 of 5 experts); layer 1:
    attention on 1 key/value head + dense feed-forward. Positions by sinusoids."""
    from liyab_amd.config import HeadSpec, LayerSpec, ModelPlan, OrderEntry, TokenEmbeddingSpec
    from liyab_amd.parts import register_ffn, register_position

    register_ffn("toy_routed", RoutedFFN)
    register_position("toy_sinusoid", SinusoidPositions)
    d, V, P, eps, E, F = 48, 157, 200, 1e-6, 5, 40
    rng = np.random.default_rng(29)
    layers = [
        LayerSpec(attention_spec("a0", d, 3, 3, 16, 0.25), RoutedSpec(d, F, E, 2, "r0"), norm_spec("n0a", d, eps), norm_spec("n0b", d, eps)),
        LayerSpec(attention_spec("a1", d, 2, 1, 32, 0.15), ffn_spec("f1", d, 72, "gelu_erf"), norm_spec("n1a", d, eps), norm_spec("n1b", d, eps)),
    ]
    tw = {"emb": rand(rng, V, d, scale=0.5), **norm_tensors(rng, "nf", d), "r0.router": rand(rng, E, d, scale=0.5),
          **attention_tensors(rng, "a0", d, 3, 3, 16), **attention_tensors(rng, "a1", d, 2, 1, 32), **ffn_tensors(rng, "f1", d, 72)}
    for e in range(E):
        tw[f"r0.{e}.up"] = rand(rng, F, d, scale=0.2)
        tw[f"r0.{e}.down"] = rand(rng, d, F, scale=0.2)
    for name in ("n0a", "n0b", "n1a", "n1b"):
        tw.update(norm_tensors(rng, name, d))
    if dtype == "bfloat16":
        tw = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v) for k, v in tw.items()}
    plan = ModelPlan(architecture="toy_routed", width=d, vocab_size=V, max_positions=P,
                     embedding=TokenEmbeddingSpec("token_embedding", V, d, 1.0, {"table": T("emb")}),
                     residual_position=SinusoidSpec(d, 50.0), layers=layers, order=[OrderEntry(0), OrderEntry(1)],
                     final_norm=norm_spec("nf", d, eps), head=HeadSpec("lm_head", d, V, 1.0, {"weight": T("emb")}))
    return plan, tw, dict(d=d, V=V, eps=eps, E=E)


def routed_plain(tw, info, ids):
    d, eps, E = info["d"], info["eps"], info["E"]
    pos = np.arange(len(ids), dtype=np.float64)[:, None]
    angle = pos / 50.0 ** (np.arange(0, d, 2, dtype=np.float64) / d)
    x = f64(tw["emb"])[ids].copy()
    x[:, 0::2] += np.sin(angle)
    x[:, 1::2] += np.cos(angle)
    a, _ = plain_attention(plain_norm(x, tw, "n0a", eps), tw, "a0", 3, 3, 16, 0.25)
    x = x + a
    h = plain_norm(x, tw, "n0b", eps)
    logits = h @ f64(tw["r0.router"]).T
    out = np.zeros_like(h)
    margins = []
    for t in range(len(ids)):
        order = np.argsort(-logits[t], kind="stable")
        chosen = order[:2]
        margins.append(logits[t, order[1]] - logits[t, order[2]])
        g = np.exp(logits[t, chosen] - logits[t, chosen].max())
        g /= g.sum()
        for gate, e in zip(g, chosen):
            out[t] += gate * (plain.gelu_tanh(h[t] @ f64(tw[f"r0.{e}.up"]).T) @ f64(tw[f"r0.{e}.down"]).T)
    x = x + out
    a, _ = plain_attention(plain_norm(x, tw, "n1a", eps), tw, "a1", 2, 1, 32, 0.15)
    x = x + a
    x = x + plain_ffn(plain_norm(x, tw, "n1b", eps), tw, "f1", "gelu_erf")
    return plain_norm(x, tw, "nf", eps) @ f64(tw["emb"]).T, np.array(margins)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_routing_and_computed_positions(dtype):
    """A feed-forward that routes and a position encoding without a table, both defined here,
    are registered, built and stepped beside the framework's attention, norms and dense
    feed-forward, under every way of cutting the work."""
    from liyab_amd.engine import EngineCore

    plan, tw, info = routed_model(dtype)
    reqs = {f"r{i}": tt.random_tokens(40 + i, n, info["V"]) for i, n in enumerate([33, 150, 2, 77])}
    ref, used = {}, set()
    for rid, toks in reqs.items():
        ref[rid], margins = routed_plain(tw, info, toks)
        if dtype == "bfloat16":
            # a token whose second and third experts are nearly tied may be routed otherwise in
            # reduced precision: such a request is cut before that token
            close = np.nonzero(margins < 0.05)[0]
            if close.size:
                reqs[rid] = toks[:max(2, int(close[0]))]
                ref[rid] = ref[rid][:len(reqs[rid])]
    assert sum(len(t) for t in reqs.values()) > 60
    tol = TOL_TOY[dtype]
    for name, steps in (("whole", tt.schedule_whole(reqs)), ("portions", tt.schedule_portions(reqs, (7, 2, 31, 3))),
                        ("mixed", tt.schedule_mixed(reqs, seed=5))):
        core = EngineCore.from_plan(plan, tw, dtype=dtype, page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=4,
                                    use_graphs=False)
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, ref, tol, f"routed toy {name} {dtype}")
        core.manager.check()
        assert all(core.manager.pages_in_use(g.index) == 0 for g in core.manager.groups)


# ---------------------------------------------------------------------------
# a toy position encoding that acts on queries and keys inside attention
# ---------------------------------------------------------------------------
class TurnSpec:
    kind = "toy_turn"
    where = "mixer"

    def __init__(self, head_dim, base):
        self.head_dim, self.base = head_dim, base


class TurnPositions:
    """Turns each pair (x[2i], x[2i + 1]) of a head by the angle pos * base^(-2i / head size): a
    test's toy in torch. It acts on the step's queries and keys where they lie, between the
    projection and the cache write, from the positions in the step's metadata."""

    where = "mixer"

    def __init__(self, spec, store, dtype):
        self.head_dim, self.base = spec.head_dim, spec.base

    def rotate(self, q, k, ctx):
        hd = self.head_dim
        i = torch.arange(0, hd, 2, device=q.device, dtype=torch.float64)
        angle = ctx.positions.double().unsqueeze(1) * self.base ** (-i / hd)  # [tokens, pairs]
        cos, sin = angle.cos().float()[:, None, :], angle.sin().float()[:, None, :]
        for x in (q, k):
            v = x.float().reshape(x.shape[0], -1, hd // 2, 2)
            a, b = v[..., 0], v[..., 1]
            x.copy_(torch.stack((a * cos - b * sin, a * sin + b * cos), dim=-1).reshape(x.shape[0], -1).to(x.dtype))


def plain_turn(x, heads, hd, base, first=0):
    """The same turn over a whole sequence whose first token stands at position `first`."""
    T_ = x.shape[0]
    angle = (first + np.arange(T_, dtype=np.float64))[:, None] * base ** (-np.arange(0, hd, 2, dtype=np.float64) / hd)
    v = x.reshape(T_, heads, hd // 2, 2)
    a, b = v[..., 0], v[..., 1]
    c, s_ = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    return np.stack((a * c - b * s_, a * s_ + b * c), axis=-1).reshape(T_, heads * hd)


def turned_model(dtype):
    """Two attention layers whose queries and keys are turned by position and no other position
    encoding: layer 0 four query heads on two key/value heads of 32, layer 1 three heads of 16
    with a window of 20 and another base."""
    import dataclasses

    from liyab_amd.config import HeadSpec, LayerSpec, ModelPlan, OrderEntry, TokenEmbeddingSpec
    from liyab_amd.parts import register_position

    register_position("toy_turn", TurnPositions)
    d, V, P, eps = 64, 190, 180, 1e-5
    rng = np.random.default_rng(41)
    a0 = dataclasses.replace(attention_spec("a0", d, 4, 2, 32, 0.2), position=TurnSpec(32, 100.0))
    a1 = dataclasses.replace(attention_spec("a1", d, 3, 3, 16, 0.3, window=20), position=TurnSpec(16, 10000.0))
    layers = [LayerSpec(a0, ffn_spec("f0", d, 96, "gelu_tanh"), norm_spec("n0a", d, eps), norm_spec("n0b", d, eps)),
              LayerSpec(a1, ffn_spec("f1", d, 80, "gelu_erf"), norm_spec("n1a", d, eps), norm_spec("n1b", d, eps))]
    tw = {"emb": rand(rng, V, d, scale=0.5), **norm_tensors(rng, "nf", d), **attention_tensors(rng, "a0", d, 4, 2, 32),
          **attention_tensors(rng, "a1", d, 3, 3, 16), **ffn_tensors(rng, "f0", d, 96), **ffn_tensors(rng, "f1", d, 80)}
    for name in ("n0a", "n0b", "n1a", "n1b"):
        tw.update(norm_tensors(rng, name, d))
    if dtype == "bfloat16":
        tw = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v) for k, v in tw.items()}
    plan = ModelPlan(architecture="toy_turned", width=d, vocab_size=V, max_positions=P,
                     embedding=TokenEmbeddingSpec("token_embedding", V, d, 1.0, {"table": T("emb")}),
                     residual_position=None, layers=layers, order=[OrderEntry(0), OrderEntry(1)],
                     final_norm=norm_spec("nf", d, eps), head=HeadSpec("lm_head", d, V, 1.0, {"weight": T("emb")}))
    return plan, tw, dict(d=d, V=V, eps=eps)


def turned_plain(tw, info, ids, first=0, turn=True):
    eps = info["eps"]
    rot = (lambda hd, base: (lambda x, heads: plain_turn(x, heads, hd, base, first))) if turn else (lambda hd, base: None)
    x = f64(tw["emb"])[ids]
    a, _ = plain_attention(plain_norm(x, tw, "n0a", eps), tw, "a0", 4, 2, 32, 0.2, rotate=rot(32, 100.0))
    x = x + a
    x = x + plain_ffn(plain_norm(x, tw, "n0b", eps), tw, "f0", "gelu_tanh")
    a, _ = plain_attention(plain_norm(x, tw, "n1a", eps), tw, "a1", 3, 3, 16, 0.3, window=20, rotate=rot(16, 10000.0))
    x = x + a
    x = x + plain_ffn(plain_norm(x, tw, "n1b", eps), tw, "f1", "gelu_erf")
    return plain_norm(x, tw, "nf", eps) @ f64(tw["emb"]).T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_position_encoding_inside_attention(dtype):
    """A position encoding that turns queries and keys, defined here, is given to the framework's
    attention as a field of its spec: it is built from the position registry and applied between
    the projection and the cache write, so a portion's keys are stored turned and later steps
    find them so. The plain formula is pinned first: only distances count (all positions moved by
    41 give the same logits), and without the turn the logits differ (the model has no other
    position encoding, so the turn is what tells positions apart)."""
    from liyab_amd.engine import EngineCore

    plan, tw, info = turned_model(dtype)
    probe = tt.random_tokens(7, 50, info["V"])
    base = turned_plain(tw, info, probe)
    assert tt.rel_err(turned_plain(tw, info, probe, first=41), base) < 1e-9
    assert tt.rel_err(turned_plain(tw, info, probe, turn=False), base) > 1e-2
    reqs = {f"p{i}": tt.random_tokens(50 + i, n, info["V"]) for i, n in enumerate([45, 180, 3, 99])}
    ref = {rid: turned_plain(tw, info, toks) for rid, toks in reqs.items()}
    for name, steps in (("whole", tt.schedule_whole(reqs)), ("portions", tt.schedule_portions(reqs, (7, 2, 31, 3, 40))),
                        ("mixed", tt.schedule_mixed(reqs, seed=8))):
        core = EngineCore.from_plan(plan, tw, dtype=dtype, page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=4)
        assert all(b.mixer.position is not None for b in core.model.blocks)
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, ref, TOL_TOY[dtype], f"turned toy {name} {dtype}", family="toy:turned")
        core.manager.check()
        assert all(core.manager.pages_in_use(g.index) == 0 for g in core.manager.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_head_without_a_norm_before_it_with_a_bias_and_a_logit_scale(dtype):
    """The plan's last two options, as data: no norm before the head (the wanted rows of the stream
    go to the product as they are) and logits times a scale, after the bias
    (src/core/transformer.cpp:2613-2620). The plain formula here is the turned toy's without its
    last norm; that bias and scale are in it shows in the difference from the unscaled one."""
    import dataclasses

    from liyab_amd.config import HeadSpec
    from liyab_amd.engine import EngineCore

    plan, tw, info = turned_model(dtype)
    scale = 0.37
    tw = {k: v for k, v in tw.items() if not k.startswith("nf.")}  # the loader refuses tensors that nobody reads
    tw["head_bias"] = rand(np.random.default_rng(77), info["V"], scale=0.5)
    plan = dataclasses.replace(plan, final_norm=None, head=HeadSpec("lm_head", info["d"], info["V"], scale,
                                                                    {"weight": T("emb"), "bias": T("head_bias")}))

    def plain_logits(ids):
        eps = info["eps"]
        rot = lambda hd, base: (lambda x, heads: plain_turn(x, heads, hd, base, 0))
        x = f64(tw["emb"])[ids]
        a, _ = plain_attention(plain_norm(x, tw, "n0a", eps), tw, "a0", 4, 2, 32, 0.2, rotate=rot(32, 100.0))
        x = x + a
        x = x + plain_ffn(plain_norm(x, tw, "n0b", eps), tw, "f0", "gelu_tanh")
        a, _ = plain_attention(plain_norm(x, tw, "n1a", eps), tw, "a1", 3, 3, 16, 0.3, window=20, rotate=rot(16, 10000.0))
        x = x + a
        x = x + plain_ffn(plain_norm(x, tw, "n1b", eps), tw, "f1", "gelu_erf")
        if dtype == "bfloat16":  # the product reads the stream in the compute dtype
            x = torch.from_numpy(x).to(torch.bfloat16).double().numpy()
        return (x @ f64(tw["emb"]).T + f64(tw["head_bias"])) * scale

    reqs = {f"h{i}": tt.random_tokens(60 + i, n, info["V"]) for i, n in enumerate([45, 130, 3, 71])}
    ref = {rid: plain_logits(toks) for rid, toks in reqs.items()}
    for name, steps in (("whole", tt.schedule_whole(reqs)), ("portions", tt.schedule_portions(reqs, (7, 2, 31, 3, 40))),
                        ("mixed", tt.schedule_mixed(reqs, seed=9))):
        core = EngineCore.from_plan(plan, tw, dtype=dtype, page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=4)
        assert core.model.final_norm is None and core.model.head.logit_scale == scale
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, ref, TOL_TOY[dtype], f"bare head {name} {dtype}", family="toy:bare_head")
        core.manager.check()


# ---------------------------------------------------------------------------
# a toy mixer that brings its own words of a step's metadata, under graphs and the scheduler
# ---------------------------------------------------------------------------
class ScanPlanner:
    """For each token, how many steps of the recurrence lie between the request's stored state
    and it (its index in the portion plus one): words of the toy mixer's own, filled on the host
    and read on the device. Nothing of them enters the key: they vary freely between replays."""

    name = "toy_scan"
    calls = 0

    def plan(self, facts):
        from liyab_amd.parts import PartStepPlan

        ScanPlanner.calls += 1
        since = np.concatenate([np.arange(1, int(n) + 1, dtype=np.int32) for n in facts.q_lens])

        def fill(address):
            import ctypes

            ctypes.memmove(address, since.ctypes.data, since.nbytes)

        return PartStepPlan(key=(), n_words=int(since.size), fill=fill, make=lambda words: words)


class PlannedDecayMixer:
    """The decay mixer again (s_t = decay * s_{t-1} + h_t, out = s_t . W^T), written so that a
    captured graph can replay it: nothing is read on the host; which request a token belongs to,
    where a request's rows end and its state slot come from the step's common metadata, and the
    distance to the stored state from the words its own planner contributes."""

    step_planner = ScanPlanner()

    def __init__(self, spec, store, dtype):
        from liyab_amd.config import TensorSource

        self.width, self.decay = spec.width, spec.decay
        self.weight = store.fetch(TensorSource(spec.prefix + ".w"), (spec.width, spec.width), "matrix")

    def cache_spec(self):
        return None

    def state_spec(self):
        from liyab_amd.cache import StateSpec

        return StateSpec((self.width,), "float32")

    def forward(self, h, ctx, cache, state, residual, writes_cache=True):
        from liyab_amd.parts import as_tensor

        h = as_tensor(h).float()
        n = h.shape[0]
        since = ctx.plans["toy_scan"].long()  # [tokens]
        seq = ctx.tok_seq.long()
        rows = torch.arange(n, device=h.device)
        gap = rows[:, None] - rows[None, :]
        mask = (seq[:, None] == seq[None, :]) & (gap >= 0)
        w = torch.pow(self.decay, gap.clamp(min=0).double()) * mask
        slots = ctx.state_slots.long()[seq]  # each token's request's slot
        carried = torch.pow(self.decay, since.double())[:, None] * state[slots].double()
        s = (w @ h.double() + carried).float()
        ends = ctx.seq_starts.long()[1:] - 1  # each request's last row
        state.index_copy_(0, ctx.state_slots.long(), s[ends])
        residual += s @ self.weight.float().t()


def planned_model():
    from liyab_amd.config import LayerSpec, OrderEntry
    from liyab_amd.parts import register_mixer

    register_mixer("toy_decay_planned", PlannedDecayMixer)
    d, V, P, eps = 48, 97, 120, 1e-5
    rng = np.random.default_rng(61)

    class Spec(DecaySpec):
        kind = "toy_decay_planned"

    layers = [LayerSpec(Spec(d, 0.7, "m0"), ffn_spec("f0", d, 64, "gelu_tanh"), norm_spec("n0a", d, eps), norm_spec("n0b", d, eps)),
              LayerSpec(attention_spec("a1", d, 3, 3, 16, 0.25), ffn_spec("f1", d, 72, "gelu_erf"), norm_spec("n1a", d, eps), norm_spec("n1b", d, eps)),
              LayerSpec(Spec(d, 0.9, "m2"), None, norm_spec("n2a", d, eps), None)]
    tw = {"emb": rand(rng, V, d, scale=0.5), "pos": rand(rng, P, d, scale=0.3), **norm_tensors(rng, "nf", d),
          "m0.w": rand(rng, d, d, scale=0.05), "m2.w": rand(rng, d, d, scale=0.05), **attention_tensors(rng, "a1", d, 3, 3, 16),
          **ffn_tensors(rng, "f0", d, 64), **ffn_tensors(rng, "f1", d, 72)}
    for name in ("n0a", "n0b", "n1a", "n1b", "n2a"):
        tw.update(norm_tensors(rng, name, d))
    return make_plan(d, V, P, layers, [OrderEntry(0), OrderEntry(1), OrderEntry(2)], eps), tw, dict(d=d, V=V, P=P, eps=eps)


def planned_plain(tw, info, ids):
    eps, d = info["eps"], info["d"]

    def decay(h, rate, w):
        s, out = np.zeros(d), np.zeros_like(h)
        for t in range(len(h)):
            s = rate * s + h[t]
            out[t] = s
        return out @ f64(tw[w]).T

    x = f64(tw["emb"])[ids] + f64(tw["pos"])[:len(ids)]
    x = x + decay(plain_norm(x, tw, "n0a", eps), 0.7, "m0.w")
    x = x + plain_ffn(plain_norm(x, tw, "n0b", eps), tw, "f0", "gelu_tanh")
    a, _ = plain_attention(plain_norm(x, tw, "n1a", eps), tw, "a1", 3, 3, 16, 0.25)
    x = x + a
    x = x + plain_ffn(plain_norm(x, tw, "n1b", eps), tw, "f1", "gelu_erf")
    x = x + decay(plain_norm(x, tw, "n2a", eps), 0.9, "m2.w")
    return plain_norm(x, tw, "nf", eps) @ f64(tw["emb"]).T


def test_a_part_with_its_own_step_metadata_runs_under_graphs_and_the_scheduler():
    """A mixer defined here keeps state of its own and has a step planner of its own: its words
    ride behind the step's common metadata, one plan a step serves both of its layers, and since
    nothing it does depends on the host it is captured and replayed like the framework's parts.
    Driven by the scheduler (portions of prompts beside decoding requests, a pool so small that
    a request is preempted and its state starts again from zero), its greedy tokens are the
    plain model's."""
    from liyab_amd import Engine, SamplingParams
    from liyab_amd.engine import EngineCore

    plan, tw, info = planned_model()
    prompts = [tt.random_tokens(70 + i, n, info["V"]) for i, n in enumerate([30, 5, 41, 17])]
    core = EngineCore.from_plan(plan, tw, dtype="float32", page_size=8, num_pages=14, max_requests=3, use_graphs=True)
    assert [p.name for p in core.model.step_planners] == ["toy_scan", "attention"]
    assert not core.step_fn.pads_rows  # the toy does not say that it takes padding rows: its steps get none
    ScanPlanner.calls = 0
    engine = Engine(core=core, max_num_seqs=3, max_batched_tokens=24, prefill_chunk=16)
    engine.stop_at_eos = False
    results = engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=30))
    assert ScanPlanner.calls == core.step_fn.steps  # once a step, not once a layer
    assert core.step_fn.graph_replays > 0
    assert any(term[0] == "toy_scan" for key in core.step_fn._graphs for term in key[3:])
    assert engine.scheduler.stats.preemptions >= 1
    for prompt, res in zip(prompts, results):
        ids, want = list(prompt), []
        for _ in range(30):
            nxt = int(np.argmax(planned_plain(tw, info, ids)[-1].astype(np.float32)))
            want.append(nxt)
            ids.append(nxt)
        assert res.tokens == want
    core.manager.check()
    assert all(core.manager.pages_in_use(g.index) == 0 for g in core.manager.groups)


# ---------------------------------------------------------------------------
# a toy mixer that keeps one narrow row a position instead of a key and a value
# ---------------------------------------------------------------------------
class NarrowSpec:
    kind = "toy_narrow"

    def __init__(self, width, rank, prefix):
        self.width, self.rank, self.prefix = width, rank, prefix


class NarrowMixer:
    """c_t = h_t . Wc^T (a row of `rank` values, the only thing cached: one plane "c" of one head);
    out_t = (mean of c_j over j <= t) . Wo^T. A test's toy in torch: it writes its rows to its own
    plane of the pages at the step's cache slots and reads a request's rows back through its
    block table, so what it keeps is paged, shared and given back like keys and values."""

    def __init__(self, spec, store, dtype):
        from liyab_amd.config import TensorSource

        self.rank = spec.rank
        self.down = store.fetch(TensorSource(spec.prefix + ".down"), (spec.rank, spec.width), "matrix")
        self.up = store.fetch(TensorSource(spec.prefix + ".up"), (spec.width, spec.rank), "matrix")

    def cache_spec(self):
        from liyab_amd.cache import KVSpec

        return KVSpec(1, self.rank, rows=(("c", 1, self.rank),))

    def state_spec(self):
        return None

    def forward(self, h, ctx, cache, state, residual, writes_cache=True):
        from liyab_amd.parts import as_tensor

        h = as_tensor(h)
        plane = cache.rows["c"]  # [pages, 1, page_size, rank]
        assert set(cache.rows) == {"c"} and plane.shape[1:] == (1, ctx.page_size, self.rank)
        group = ctx.groups[cache.group]
        c = (h.float() @ self.down.float().t()).to(plane.dtype)
        flat = plane.view(-1, self.rank)  # one head: slot = page * page_size + offset indexes rows directly
        if writes_cache:
            flat.index_copy_(0, group.slots.long(), c)
        out = torch.empty(h.shape[0], self.rank, device=h.device)
        tables = group.block_tables.tolist()
        for i, (a, n, first) in enumerate(zip(ctx.host.starts, ctx.host.q_lens, ctx.host.first_pos)):
            length = first + n
            pages = torch.tensor(tables[i][:-(-length // ctx.page_size)], device=h.device)
            kept = plane[pages, 0].reshape(-1, self.rank)[:length].float()
            means = kept.cumsum(0) / torch.arange(1, length + 1, device=h.device)[:, None]
            out[a:a + n] = means[first:]
        residual += out @ self.up.float().t()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_mixer_with_rows_of_its_own_in_the_pages(dtype):
    """The pages of a group hold whatever planes of rows its mixers name: here one row of 24
    values a position beside an attention layer's keys and values of 5 heads of 16 (two groups,
    each with its pages and block tables). Whole, in portions and mixed with few pages."""
    from liyab_amd.config import LayerSpec, OrderEntry
    from liyab_amd.engine import EngineCore
    from liyab_amd.parts import register_mixer

    register_mixer("toy_narrow", NarrowMixer)
    d, V, P, eps, r = 80, 150, 140, 1e-5, 24
    rng = np.random.default_rng(73)
    layers = [LayerSpec(NarrowSpec(d, r, "m0"), ffn_spec("f0", d, 96, "gelu_tanh"), norm_spec("n0a", d, eps), norm_spec("n0b", d, eps)),
              LayerSpec(attention_spec("a1", d, 5, 5, 16, 0.25), None, norm_spec("n1a", d, eps), None)]
    tw = {"emb": rand(rng, V, d, scale=0.5), "pos": rand(rng, P, d, scale=0.3), **norm_tensors(rng, "nf", d),
          "m0.down": rand(rng, r, d, scale=0.2), "m0.up": rand(rng, d, r, scale=0.2), **attention_tensors(rng, "a1", d, 5, 5, 16),
          **ffn_tensors(rng, "f0", d, 96), **norm_tensors(rng, "n0a", d), **norm_tensors(rng, "n0b", d), **norm_tensors(rng, "n1a", d)}
    if dtype == "bfloat16":
        tw = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v) for k, v in tw.items()}
    plan = make_plan(d, V, P, layers, [OrderEntry(0), OrderEntry(1)], eps)

    def plain_model(ids):
        x = f64(tw["emb"])[ids] + f64(tw["pos"])[:len(ids)]
        c = plain_norm(x, tw, "n0a", eps) @ f64(tw["m0.down"]).T
        means = np.cumsum(c, axis=0) / np.arange(1, len(ids) + 1)[:, None]
        x = x + means @ f64(tw["m0.up"]).T
        x = x + plain_ffn(plain_norm(x, tw, "n0b", eps), tw, "f0", "gelu_tanh")
        a, _ = plain_attention(plain_norm(x, tw, "n1a", eps), tw, "a1", 5, 5, 16, 0.25)
        return plain_norm(x + a, tw, "nf", eps) @ f64(tw["emb"]).T

    reqs = {f"n{i}": tt.random_tokens(20 + i, n, V) for i, n in enumerate([50, 140, 4, 77])}
    ref = {rid: plain_model(toks) for rid, toks in reqs.items()}
    for name, steps in (("whole", tt.schedule_whole(reqs)), ("portions", tt.schedule_portions(reqs, (7, 2, 31, 3))),
                        ("mixed", tt.schedule_mixed(reqs, seed=6))):
        core = EngineCore.from_plan(plan, tw, dtype=dtype, page_size=8, max_tokens=tt.max_live_tokens(steps), max_requests=4,
                                    use_graphs=False)  # the toy reads block tables on the host
        assert sorted(g.spec.planes for g in core.manager.groups) == [(("c", 1, r),), (("k", 5, 16), ("v", 5, 16))]
        assert core.storage.bytes_per_token() == (r + 2 * 5 * 16) * (4 if dtype == "float32" else 2)
        for c in core.storage.layers.values():
            for t in c.rows.values():
                t.fill_(float("nan"))
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, ref, TOL_TOY[dtype], f"narrow toy {name} {dtype}", family="toy:narrow")
        core.manager.check()
        assert all(core.manager.pages_in_use(g.index) == 0 for g in core.manager.groups)


class BareNorm:
    """A LayerNorm that knows nothing of split streams or pending norms (no `takes_planes`, no `lazy`)."""

    def __init__(self, spec, store, dtype):
        self.width, self.eps, self.dtype = spec.width, float(spec.eps), dtype
        self.weight = store.fetch(spec.tensors["weight"], (self.width,), "vector")
        self.bias = store.fetch(spec.tensors["bias"], (self.width,), "vector")

    def forward(self, x, ctx, rows=None, n_rows=None, name="normed"):
        from liyab_amd.kernels import ops

        n = x.shape[0] if rows is None else (n_rows if n_rows is not None else rows.numel())
        out = ctx.workspace.get(name, (n, self.width), self.dtype)
        ops.layernorm(out, x, self.weight, self.bias, self.eps, rows=rows)
        return out


class BareBlock:
    """The pre-norm arrangement written without any of the optional interfaces."""

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn):
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn

    def forward(self, x, ctx, cache, state, writes_cache=True):
        self.mixer.forward(self.norm_mixer.forward(x, ctx), ctx, cache, state, x, writes_cache=writes_cache)
        if self.ffn is not None:
            self.ffn.forward(self.norm_ffn.forward(x, ctx), ctx, x)


def test_split_streams_reach_parts_that_cannot_take_them(monkeypatch):
    """Products cut over K leave the residual stream split into planes for its next reader.
    Here the cut is forced at the toy model's small sizes; layer 1's second norm (after the
    attention whose projection is cut) is one that cannot read planes, and layer 2's block
    (after layer 1's cut feed-forward) one that cannot take a split stream: the planes are
    added up before those parts run; the last layer's go to the final norm over gathered rows;
    the logits stay those of the plain model."""
    import dataclasses

    from liyab_amd.engine import EngineCore
    from liyab_amd.kernels import ops
    from liyab_amd.parts import register_block, register_norm

    register_norm("bare_layernorm", BareNorm)
    register_block("bare_pre_norm", BareBlock)
    cut = []

    def forced(M, N, K):
        parts = 2 if M <= 16 and K % 8 == 0 and K > 64 else 1
        cut.append(parts)
        return parts

    monkeypatch.setattr(ops, "k_parts", forced)
    plan, tw, info = toy_model("bfloat16")
    layers = list(plan.layers)
    layers[1] = dataclasses.replace(layers[1], norm_ffn=dataclasses.replace(layers[1].norm_ffn, kind="bare_layernorm"))
    layers[2] = dataclasses.replace(layers[2], arrangement="bare_pre_norm")
    plan = dataclasses.replace(plan, layers=layers)
    reqs = {f"t{i}": tt.random_tokens(90 + i, n, info["V"]) for i, n in enumerate([37, 90, 5, 61])}
    ref = {rid: toy_plain(tw, info, toks) for rid, toks in reqs.items()}
    for name, steps in (("portions", tt.schedule_portions(reqs, (5, 2, 11, 3, 16))), ("mixed", tt.schedule_mixed(reqs, seed=3))):
        core = EngineCore.from_plan(plan, tw, dtype="bfloat16", page_size=8, max_tokens=tt.max_live_tokens(steps), max_requests=4,
                                    use_graphs=False)
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, ref, TOL_TOY["bfloat16"], f"toy with forced cuts, {name}")
        core.manager.check()
    assert 2 in cut and 1 in cut  # both ways were taken


# ---------------------------------------------------------------------------
# another norm and two other arrangements of a block
# ---------------------------------------------------------------------------
class RmsSpec:
    kind = "toy_rms"

    def __init__(self, width, eps, prefix):
        self.width, self.eps, self.prefix = width, eps, prefix


class RmsNorm:
    """y = x / sqrt(mean(x^2) + eps) * weight: no mean taken off, no bias. A test's toy in torch with
    only what a norm must have: forward(x, ctx, rows, n_rows, name) -> rows in the compute dtype."""

    def __init__(self, spec, store, dtype):
        from liyab_amd.config import TensorSource

        self.width, self.eps, self.dtype = spec.width, float(spec.eps), dtype
        self.weight = store.fetch(TensorSource(spec.prefix + ".w"), (self.width,), "vector")

    def forward(self, x, ctx, rows=None, n_rows=None, name="normed"):
        x = x.float()
        if rows is not None:
            x = x[rows.long()[:n_rows if n_rows is not None else rows.numel()]]
        out = ctx.workspace.get(name, tuple(x.shape), self.dtype)
        out.copy_(self.stream(x))
        return out

    def stream(self, x):
        """The same in 32-bit, for a block that keeps the norm's output as the stream."""
        return x * torch.rsqrt((x * x).mean(dim=1, keepdim=True) + self.eps) * self.weight.float()


class ParallelBlock:
    """x += mixer(norm(x)) + ffn(norm(x)): one norm, both parts read its rows."""

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn):
        assert norm_ffn is None
        self.mixer, self.ffn, self.norm = mixer, ffn, norm_mixer

    def forward(self, x, ctx, cache, state, writes_cache=True):
        h = self.norm.forward(x, ctx, name="parallel_in").clone()  # (both parts read it: not the workspace's next view of that name)
        self.mixer.forward(h, ctx, cache, state, x, writes_cache=writes_cache)
        self.ffn.forward(h, ctx, x)


class PostNormBlock:
    """x = norm_mixer(x + mixer(x)); x = norm_ffn(x + ffn(x)): the norms come after the sums and
    the stream itself is what they leave."""

    def __init__(self, spec, mixer, ffn, norm_mixer, norm_ffn):
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn
        self.dtype = mixer.dtype

    def forward(self, x, ctx, cache, state, writes_cache=True):
        self.mixer.forward(x.to(self.dtype), ctx, cache, state, x, writes_cache=writes_cache)
        x.copy_(self.norm_mixer.stream(x))
        self.ffn.forward(x.to(self.dtype), ctx, x)
        x.copy_(self.norm_ffn.stream(x))


def arranged_model(dtype="float32"):
    """Layer 0: a parallel block behind the framework's LayerNorm (4 query heads on 2 key/value heads
    of 16, tanh feed-forward); layer 1: a post-norm block with root-mean-square norms (3 heads of 32,
    erf feed-forward); the final norm is the toy's too."""
    from liyab_amd.config import HeadSpec, LayerSpec, ModelPlan, OrderEntry, PositionSpec, TokenEmbeddingSpec
    from liyab_amd.parts import register_block, register_norm

    register_norm("toy_rms", RmsNorm)
    register_block("toy_parallel", ParallelBlock)
    register_block("toy_post_norm", PostNormBlock)
    d, V, P, eps = 96, 211, 160, 2e-5
    rng = np.random.default_rng(31)
    layers = [
        LayerSpec(attention_spec("a0", d, 4, 2, 16, 0.3), ffn_spec("f0", d, 120, "gelu_tanh"), norm_spec("n0", d, eps), None, arrangement="toy_parallel"),
        LayerSpec(attention_spec("a1", d, 3, 3, 32, 0.05), ffn_spec("f1", d, 88, "gelu_erf"), RmsSpec(d, eps, "r1a"), RmsSpec(d, eps, "r1b"),
                  arrangement="toy_post_norm"),
    ]
    tw = {"emb": rand(rng, V, d, scale=0.5), "pos": rand(rng, P, d, scale=0.3), "r1a.w": rand(rng, d, scale=0.1, mean=1.0),
          "r1b.w": rand(rng, d, scale=0.1, mean=1.0), "rf.w": rand(rng, d, scale=0.1, mean=1.0), **norm_tensors(rng, "n0", d),
          **attention_tensors(rng, "a0", d, 4, 2, 16), **attention_tensors(rng, "a1", d, 3, 3, 32),
          **ffn_tensors(rng, "f0", d, 120), **ffn_tensors(rng, "f1", d, 88)}
    if dtype == "bfloat16":
        tw = {k: (v.to(torch.bfloat16).float() if v.dim() == 2 else v) for k, v in tw.items()}
    plan = ModelPlan(architecture="toy_arranged", width=d, vocab_size=V, max_positions=P,
                     embedding=TokenEmbeddingSpec("token_embedding", V, d, 1.0, {"table": T("emb")}),
                     residual_position=PositionSpec("learned_positions", "residual", P, d, {"table": T("pos")}),
                     layers=layers, order=[OrderEntry(0), OrderEntry(1)], final_norm=RmsSpec(d, eps, "rf"),
                     head=HeadSpec("lm_head", d, V, 1.0, {"weight": T("emb")}))
    return plan, tw, dict(d=d, V=V, eps=eps)


def arranged_plain(tw, info, ids):
    eps = info["eps"]

    def rms(x, name):
        return x / np.sqrt((x * x).mean(axis=1, keepdims=True) + eps) * f64(tw[name + ".w"])

    x = f64(tw["emb"])[ids] + f64(tw["pos"])[:len(ids)]
    h = plain_norm(x, tw, "n0", eps)
    a, _ = plain_attention(h, tw, "a0", 4, 2, 16, 0.3)
    x = x + a + plain_ffn(h, tw, "f0", "gelu_tanh")
    a, _ = plain_attention(x, tw, "a1", 3, 3, 32, 0.05)  # (it reads the stream as it is, several units large: a small scale keeps the scores moderate)
    x = rms(x + a, "r1a")
    x = rms(x + plain_ffn(x, tw, "f1", "gelu_erf"), "r1b")
    return rms(x, "rf") @ f64(tw["emb"]).T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_norm_and_other_arrangements_of_a_block(dtype):
    """A root-mean-square norm, a parallel block and a post-norm block, all defined here, are
    registered and built around the framework's attention and feed-forward and stepped under every
    way of cutting the work: the norm's kind, where it stands and what the stream holds between the
    parts belong to the plan, not to the model class. (The parts here say nothing of padding rows, split
    streams or recorded lists: the engine then pads nothing, adds planes up first and runs their Python.)"""
    from liyab_amd.engine import EngineCore

    plan, tw, info = arranged_model(dtype)
    reqs = {f"p{i}": tt.random_tokens(60 + i, n, info["V"]) for i, n in enumerate([35, 160, 3, 81])}
    ref = {rid: arranged_plain(tw, info, toks) for rid, toks in reqs.items()}
    # (a plausible mistake fails it: a mean taken off in the toy norm, or the second part reading the stream
    # after the first has added to it, moves the logits by far more than the tolerance)
    x = f64(tw["emb"])[reqs["p0"]] + f64(tw["pos"])[:35]
    assert tt.rel_err((x - x.mean(axis=1, keepdims=True)) @ f64(tw["emb"]).T, x @ f64(tw["emb"]).T) > 1e-2
    for name, steps in (("whole", tt.schedule_whole(reqs)), ("portions", tt.schedule_portions(reqs, (7, 2, 31, 3))),
                        ("mixed", tt.schedule_mixed(reqs, seed=7))):
        for use_graphs in (False, True):
            core = EngineCore.from_plan(plan, tw, dtype=dtype, page_size=16, max_tokens=tt.max_live_tokens(steps), max_requests=4,
                                        use_graphs=use_graphs)
            assert not core.step_fn.pads_rows and core.model.replayed_layers == 0
            got = tt.run_schedule(core, steps)
            tt.check_against_plain(got, reqs, ref, TOL_TOY[dtype], f"arranged toy {name} {dtype}")
            assert core.model.replayed_layers == 0
            core.manager.check()
            assert all(core.manager.pages_in_use(g.index) == 0 for g in core.manager.groups)


# ---------------------------------------------------------------------------
# a whole architecture of a test's own, from its config.json to greedy tokens
# ---------------------------------------------------------------------------
class ToyWindowConfig:
    """An architecture of this test's own: config.json keys of its own, a plan made of the
    package's parts in a mix GPT-2 has not: layers alternate between attention over all keys and
    grouped attention over a window (two cache groups), the head is a matrix of its own with a bias,
    the feed-forward's width and activation alternate too. Nothing of it is in the package's files."""

    architecture = "ToyWindowLM"

    def __init__(self, raw):
        self.raw = dict(raw)
        for key in ("layers", "width", "heads", "kv_heads", "inner", "vocab", "positions", "window"):
            if not isinstance(raw.get(key), int) or raw[key] <= 0:
                from liyab_amd.errors import InvalidModel

                raise InvalidModel(f"missing or invalid {key}")
        self.eps = float(raw.get("eps", 1e-5))

    @classmethod
    def from_json(cls, raw):
        return cls(raw)

    def to_json(self):
        return dict(self.raw, architectures=[self.architecture])

    def plan(self):
        from liyab_amd.config import (AttentionSpec, DenseFFNSpec, HeadSpec, LayerSpec, ModelPlan, NormSpec, OrderEntry, PositionSpec,
                                      TensorSource, TokenEmbeddingSpec)
        from liyab_amd.config.plan import Init

        r = self.raw
        d, H, V, P = r["width"], r["heads"], r["vocab"], r["positions"]
        hd = d // H
        small, unit = Init(0.08), Init(0.05, 1.0)

        def norm(name):
            return NormSpec("layernorm", d, self.eps, {"weight": TensorSource(name + ".gain", init=unit), "bias": TensorSource(name + ".shift", init=small)})

        layers = []
        for i in range(r["layers"]):
            windowed = i % 2 == 1
            Hkv = r["kv_heads"] if windowed else H
            p = f"blocks.{i}"
            mixer = AttentionSpec("attention", d, H, Hkv, hd, 1.0 / math.sqrt(hd), r["window"] if windowed else 0,
                                  {"qkv_weight": TensorSource(p + ".qkv", init=small), "qkv_bias": TensorSource(p + ".qkv_b", init=small),
                                   "out_weight": TensorSource(p + ".out", init=small), "out_bias": TensorSource(p + ".out_b", init=small)})
            F = r["inner"] + 16 * (i % 2)
            ffn = DenseFFNSpec("dense_ffn", d, F, "gelu_erf" if windowed else "gelu_tanh",
                               {"up_weight": TensorSource(p + ".up", init=small), "up_bias": TensorSource(p + ".up_b", init=small),
                                "down_weight": TensorSource(p + ".down", init=small), "down_bias": TensorSource(p + ".down_b", init=small)})
            layers.append(LayerSpec(mixer, ffn, norm(p + ".norm_a"), norm(p + ".norm_f")))
        return ModelPlan(architecture=self.architecture, width=d, vocab_size=V, max_positions=P,
                         embedding=TokenEmbeddingSpec("token_embedding", V, d, 1.0, {"table": TensorSource("tokens", init=Init(0.3))}),
                         residual_position=PositionSpec("learned_positions", "residual", P, d, {"table": TensorSource("places", init=Init(0.2))}),
                         layers=layers, order=[OrderEntry(i) for i in range(r["layers"])], final_norm=norm("norm_out"),
                         head=HeadSpec("lm_head", d, V, 1.0, {"weight": TensorSource("unembed", init=Init(0.1)), "bias": TensorSource("unembed_b", init=small)}))


def toy_window_plain(raw, t, ids):
    """The toy architecture's logits for a whole sequence, float64, from the folder's tensors by name."""
    d, H, eps = raw["width"], raw["heads"], float(raw.get("eps", 1e-5))
    hd = d // H
    x = t["tokens"][ids] + t["places"][:len(ids)]
    for i in range(raw["layers"]):
        windowed = i % 2 == 1
        Hkv = raw["kv_heads"] if windowed else H
        p = f"blocks.{i}"
        h = plain.layer_norm(x, t[p + ".norm_a.gain"], t[p + ".norm_a.shift"], eps)
        qkv = h @ t[p + ".qkv"].T + t[p + ".qkv_b"]
        q, k, v = qkv[:, :H * hd], qkv[:, H * hd:(H + Hkv) * hd], qkv[:, (H + Hkv) * hd:]
        rep = H // Hkv
        kk = np.concatenate([k[:, (hh // rep) * hd:(hh // rep + 1) * hd] for hh in range(H)], axis=1)
        vv = np.concatenate([v[:, (hh // rep) * hd:(hh // rep + 1) * hd] for hh in range(H)], axis=1)
        x = x + plain.causal_attention(q, kk, vv, H, 1.0 / math.sqrt(hd), raw["window"] if windowed else 0) @ t[p + ".out"].T + t[p + ".out_b"]
        h = plain.layer_norm(x, t[p + ".norm_f.gain"], t[p + ".norm_f.shift"], eps)
        act = plain.gelu_erf if windowed else plain.gelu_tanh
        x = x + act(h @ t[p + ".up"].T + t[p + ".up_b"]) @ t[p + ".down"].T + t[p + ".down_b"]
    return plain.layer_norm(x, t["norm_out.gain"], t["norm_out.shift"], eps) @ t["unembed"].T + t["unembed_b"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_an_architecture_of_the_tests_own_from_config_json_to_greedy_tokens(dtype, tmp_path):
    """What adding an architecture takes: a configuration class (from_json, to_json, plan) and one call
    of register_architecture, here from a test. From then on the name in config.json finds it: the
    random-weights mode writes its folder from the plan's tensor names and rules, the loader reads it back by
    name (and says what is missing when a tensor is taken out), the cache manager gives its two kinds of layers
    groups of pages of their own, the step function runs it whole, in portions and mixed under graphs, and the
    engine's loop generates greedy tokens with it; all against a plain implementation written here."""
    from safetensors import safe_open
    from safetensors.torch import save_file

    from liyab_amd import Engine, InvalidModel, SamplingParams, Unsupported
    from liyab_amd.config import register_architecture
    from liyab_amd.config.registry import load_config
    from liyab_amd.engine import EngineCore
    from liyab_amd.weights import write_random_model

    raw = {"architectures": ["ToyWindowLM"], "layers": 3, "width": 96, "heads": 6, "kv_heads": 2, "inner": 136, "vocab": 333,
           "positions": 200, "window": 40, "eps": 3e-5}
    register_architecture("ToyWindowLM", ToyWindowConfig)
    folder = write_random_model(str(tmp_path / "model"), raw, seed=4)
    assert isinstance(load_config(folder), ToyWindowConfig)
    with pytest.raises(Unsupported, match="ToyWindowLM"):  # the list of what is supported names it now
        load_config(write_bad_config(tmp_path / "other", {"architectures": ["NoSuchLM"]}))
    with pytest.raises(InvalidModel, match="missing or invalid kv_heads"):
        load_config(write_bad_config(tmp_path / "incomplete", {k: v for k, v in raw.items() if k != "kv_heads"}))
    config, tensors = plain.read_model(folder)
    assert tensors["blocks.1.qkv"].shape == ((6 + 2 * 2) * 16, 96) and tensors["blocks.0.up"].shape == (136, 96) and tensors["blocks.1.up"].shape == (152, 96)
    if dtype == "bfloat16":
        tensors = plain.round_weights_to_bf16(tensors)
    reqs = {f"w{i}": tt.random_tokens(20 + i, n, raw["vocab"]) for i, n in enumerate([200, 47, 3, 120])}
    ref = {rid: toy_window_plain(raw, tensors, toks) for rid, toks in reqs.items()}
    for name, steps in (("whole", tt.schedule_whole(reqs)), ("portions", tt.schedule_portions(reqs)), ("mixed", tt.schedule_mixed(reqs, seed=9))):
        core = EngineCore(folder, dtype=dtype, page_size=8, max_tokens=tt.max_live_tokens(steps), max_requests=4, use_graphs=True)
        assert sorted(g.spec.window for g in core.manager.groups) == [0, 40] and [len(g.layers) for g in core.manager.groups if g.spec.window == 0] == [2]
        got = tt.run_schedule(core, steps)
        tt.check_against_plain(got, reqs, ref, TOL[dtype], f"architecture {name} {dtype}", family="toy:architecture")
        core.manager.check()
        del core
    # greedy tokens through the engine's loop and the scheduler
    prompts = [reqs["w1"], reqs["w2"], reqs["w3"][:60]]
    engine = Engine(folder, dtype=dtype, page_size=8, max_num_seqs=3, max_batched_tokens=48, prefill_chunk=32)
    engine.stop_at_eos = False
    for prompt, res in zip(prompts, engine.generate(prompts, SamplingParams(temperature=0.0, max_tokens=16))):
        assert len(res.tokens) == 16
        rows = toy_window_plain(raw, tensors, prompt + res.tokens[:-1])[len(prompt) - 1:]
        tol = 1e-5 if dtype == "float32" else TOL[dtype]
        assert all(row[tok] >= row.max() - tol * np.abs(row).max() for row, tok in zip(rows, res.tokens))
    # a folder with a tensor taken out: one error that names it
    kept = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for key in f.keys():
            if key != "blocks.2.norm_f.shift":
                kept[key] = f.get_tensor(key)
    broken = tmp_path / "broken"
    broken.mkdir()
    save_file(kept, str(broken / "model.safetensors"))
    (broken / "config.json").write_text((tmp_path / "model" / "config.json").read_text())
    with pytest.raises(InvalidModel, match="blocks.2.norm_f.shift"):
        EngineCore(str(broken), dtype=dtype, page_size=8, max_tokens=64, max_requests=2)


def write_bad_config(folder, raw):
    import json

    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(raw))
    return str(folder)


def test_unknown_kinds_are_refused_by_name():
    from liyab_amd import Unsupported
    from liyab_amd.config import LayerSpec, OrderEntry
    from liyab_amd.engine import EngineCore

    class Nameless:
        kind = "no_such_mixer"

    plan, tw, info = toy_model()
    bad = LayerSpec(Nameless(), None, norm_spec("n0a", info["d"], 1e-5), None)
    with pytest.raises(Unsupported, match="mixer kind 'no_such_mixer' is not registered"):
        EngineCore.from_plan(make_plan(info["d"], info["V"], info["P"], [bad], [OrderEntry(0)]), tw)
