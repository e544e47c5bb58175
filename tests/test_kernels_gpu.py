"""Each kernel alone against a plain 32-bit PyTorch reference of the same operation, at
sizes other than the engine's (needs the GPU)."""

import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from liyab_amd.kernels import ops as o

    o.check_device()
    return o


def rnd(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype).to(DEV)


def close(got, want, tol, what=""):
    got, want = got.double().cpu(), want.double().cpu()
    err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-30)
    assert math.isfinite(err) and err <= tol, f"{what}: relative error {err:.3e} > {tol:.1e}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,d", [(1, 64), (7, 100), (33, 1600), (5, 4096 + 24), (3, 4096), (2, 777), (4, 8200), (9, 768)])
def test_embed_and_add_rows(ops, dtype, n, d):
    V, P = 321, 77
    table, pos = rnd(V, d, dtype=dtype), rnd(P, d, dtype=dtype, seed=1)
    ids = torch.randint(0, V, (n,), dtype=torch.int32, device=DEV)
    positions = torch.randint(0, P, (n,), dtype=torch.int32, device=DEV)
    out = torch.empty(n, d, device=DEV)
    ops.embed(out, table, ids, 1.0, pos_table=pos, positions=positions)
    want = table.float()[ids.long()] + pos.float()[positions.long()]
    assert torch.equal(out, want)
    ops.embed(out, table, ids, 2.5)
    assert torch.equal(out, table.float()[ids.long()] * 2.5)
    ops.add_rows_(out, pos, positions)
    assert torch.equal(out, table.float()[ids.long()] * 2.5 + pos.float()[positions.long()])


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,d,eps", [(1, 64, 1e-5), (9, 96, 1e-6), (40, 1600, 1e-5), (3, 777, 1e-3), (5, 768, 1e-5),
                                     (70, 260, 1e-5), (6, 1028, 1e-6), (7, 2048, 1e-5), (2, 2052, 1e-5), (4, 4096, 1e-5), (3, 5120, 1e-6),
                                     (2, 16384, 1e-5), (2, 16388, 1e-5), (3, 4098, 1e-5)])
def test_layernorm(ops, out_dtype, n, d, eps):
    x = rnd(n + 3, d, scale=3.0) + 1.5
    w, b = rnd(d, seed=2) + 1.0, rnd(d, seed=3)
    out = torch.empty(n, d, dtype=out_dtype, device=DEV)
    ops.layernorm(out, x, w, b, eps)
    want = torch.nn.functional.layer_norm(x[:n].double(), (d,), w.double(), b.double(), eps)
    close(out, want, 1e-6 if out_dtype == torch.float32 else 5e-3, "layernorm")
    rows = torch.tensor([(i * 2) % (n + 3) for i in range(n)], dtype=torch.int32, device=DEV)
    ops.layernorm(out, x, w, None, eps, rows=rows)
    want = torch.nn.functional.layer_norm(x[rows.long()].double(), (d,), w.double(), None, eps)
    close(out, want, 1e-6 if out_dtype == torch.float32 else 5e-3, "layernorm gather")
    # eps is the kernel's argument, not a constant: a low-variance row shows it
    flat = torch.ones(1, d, device=DEV) + 1e-3 * rnd(1, d, seed=9)
    o1, o2 = torch.empty(1, d, device=DEV), torch.empty(1, d, device=DEV)
    ops.layernorm(o1, flat, None, None, 1e-5)
    ops.layernorm(o2, flat, None, None, 1e-6)
    assert (o1 - o2).abs().max() > 1e-2


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,d,parts", [(1, 64, 1), (9, 96, 4), (16, 768, 4), (5, 1600, 2), (7, 2048, 5), (6, 200, 16), (70, 768, 3),
                                       (5, 4096, 3), (2, 8192, 4), (3, 2052, 2)])
def test_layernorm_over_rows_in_planes(ops, out_dtype, n, d, parts):
    """Rows given as a sum of planes: the norm adds the planes up, in their order, as it loads a
    row, also over gathered rows; sum_parts alone does the same sum (into a tensor of its own or
    into the first plane); widths the kernel does not take in planes are refused."""
    tol = 1e-6 if out_dtype == torch.float32 else 5e-3
    planes = rnd(parts, n + 3, d, seed=4, scale=0.7)
    planes[0] += 1.5
    w, b = rnd(d, seed=2) + 1.0, rnd(d, seed=3)
    total = planes.double().sum(0)
    want = torch.nn.functional.layer_norm(total, (d,), w.double(), b.double(), 1e-5)
    out = torch.empty(n, d, dtype=out_dtype, device=DEV)
    before = planes.clone()
    ops.layernorm(out, planes, w, b, 1e-5)
    close(out, want[:n], tol, "layernorm over planes")
    assert torch.equal(planes, before)  # the planes stay as they are
    summed = torch.empty(n + 3, d, device=DEV)
    ops.sum_parts(summed, planes)
    close(summed, total, 1e-6, "sum of the planes")
    whole = torch.empty(n, d, dtype=out_dtype, device=DEV)
    ops.layernorm(whole, summed, w, b, 1e-5)
    assert torch.equal(whole, out)  # the same order of additions
    rows = torch.tensor([(i * 3) % (n + 3) for i in range(n + 2)], dtype=torch.int32, device=DEV)  # names rows twice
    out = torch.empty(n + 2, d, dtype=out_dtype, device=DEV)
    ops.layernorm(out, planes, w, b, 1e-5, rows=rows)
    close(out, want[rows.long()], tol, "gathered layernorm over planes")
    ops.sum_parts(planes[0], planes)
    assert torch.equal(planes[0], summed)
    if parts > 1:
        odd = rnd(parts, 3, 777, seed=6)
        assert not ops.norm_takes_planes(777)
        with pytest.raises(Exception, match="planes"):
            ops.layernorm(torch.empty(3, 777, device=DEV), odd, rnd(777), rnd(777), 1e-5)
    with pytest.raises(Exception, match="rows of d"):
        ops.layernorm(torch.empty(n, d, device=DEV), planes[:, :, :-4].contiguous(), w, b, 1e-5)


@pytest.mark.parametrize("M,N,K,parts", [(1, 64, 128, 2), (8, 768, 3072, 4), (16, 100, 200, 2), (5, 1600, 6400, 2), (40, 50, 448, 7),
                                         (64, 264, 1600, 3), (3, 40, 64, 1), (11, 130, 1032, 4)])
def test_gemm_skinny_parts(ops, M, N, K, parts):
    """The product cut over K: plane p holds the sums over the p-th part of K (whole units of
    64, the last one shorter); the planes add up to the product. With rows to add to (a tensor
    or planes of their own), the first plane also takes them and the bias, and the planes add
    up to rows + product + bias."""
    a, w = rnd(M, K, dtype=torch.bfloat16), rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16)
    planes = torch.full((parts, M, N), float("nan"), device=DEV)
    ops.gemm_skinny_parts(a, w, planes)
    units = (K + 63) // 64
    part_k = (units + parts - 1) // parts * 64
    for q in range(parts):
        lo, hi = q * part_k, min(K, (q + 1) * part_k)
        close(planes[q], a[:, lo:hi].double() @ w[:, lo:hi].double().t(), 1e-5, f"part {q}")
    product = a.double() @ w.double().t()
    close(planes.sum(0), product, 1e-5, "sum of the parts")
    bias = rnd(N, seed=7)
    for n_base in (0, 1, 3, 6):
        base = rnd(M, N, seed=8, scale=3.0) if n_base == 0 else rnd(n_base, M, N, seed=9, scale=3.0)
        for with_bias in (True, False):
            based = torch.full((parts, M, N), float("nan"), device=DEV)
            ops.gemm_skinny_parts(a, w, based, bias=bias if with_bias else None, base=base)
            assert torch.equal(based[1:], planes[1:])
            rows = base.double() if n_base == 0 else base.double().sum(0)
            want0 = planes[0].double() + rows + (bias.double() if with_bias else 0)
            close(based[0], want0, 1e-6, f"first plane over {n_base} planes of rows")
            close(based.double().sum(0), product + rows + (bias.double() if with_bias else 0), 1e-5, "sum with rows")
    with pytest.raises(Exception, match="parts"):
        ops.gemm_skinny_parts(a, w, torch.empty(K // 64 + 2, M, N, device=DEV))
    with pytest.raises(Exception, match="bias needs"):
        ops.gemm_skinny_parts(a, w, planes, bias=bias)
    with pytest.raises(Exception, match="overlap"):
        ops.gemm_skinny_parts(a, w, planes, base=planes[:1])


@pytest.mark.parametrize("tile", [6, 16, 17])
@pytest.mark.parametrize("M,N,K,parts", [(64, 768, 3072, 4), (2048, 768, 3072, 2), (200, 100, 448, 3), (33, 1600, 6400, 4), (1, 40, 64, 1),
                                         (130, 777, 1088, 5)])
def test_gemm_tiled_parts(ops, tile, M, N, K, parts):
    """The tiled product cut over K: plane p holds the sums over the p-th part of K (whole tiles
    of 64); with rows to add to, the first plane also takes them and the bias."""
    a, w = rnd(M, K, dtype=torch.bfloat16), rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16)
    planes = torch.full((parts, M, N), float("nan"), device=DEV)
    ops.gemm_mfma_dl_parts(a, w, planes, tile=tile)
    part_k = (K // 64 + parts - 1) // parts * 64
    for q in range(parts):
        lo, hi = q * part_k, min(K, (q + 1) * part_k)
        close(planes[q], a[:, lo:hi].double() @ w[:, lo:hi].double().t(), 1e-5, f"part {q}")
    product = a.double() @ w.double().t()
    bias = rnd(N, seed=7)
    for n_base in (0, 3):
        base = rnd(M, N, seed=8, scale=3.0) if n_base == 0 else rnd(n_base, M, N, seed=9, scale=3.0)
        for with_bias in (True, False):
            based = torch.full((parts, M, N), float("nan"), device=DEV)
            ops.gemm_mfma_dl_parts(a, w, based, bias=bias if with_bias else None, base=base, tile=tile)
            assert torch.equal(based[1:], planes[1:])
            rows = base.double() if n_base == 0 else base.double().sum(0)
            close(based[0], planes[0].double() + rows + (bias.double() if with_bias else 0), 1e-6, f"first plane over {n_base} planes of rows")
            close(based.double().sum(0), product + rows + (bias.double() if with_bias else 0), 1e-5, "sum with rows")
    with pytest.raises(Exception, match="parts"):
        ops.gemm_mfma_dl_parts(a, w, torch.empty(K // 64 + 2, M, N, device=DEV), tile=tile)
    with pytest.raises(Exception, match="overlap"):
        ops.gemm_mfma_dl_parts(a, w, planes, base=planes[:1], tile=tile)


def gemm_reference(a, w, bias, epilogue, residual=None):
    y = a.double() @ w.double().t()
    if bias is not None:
        y = y + bias.double()
    if epilogue == "gelu_tanh":
        y = torch.nn.functional.gelu(y, approximate="tanh")
    elif epilogue == "gelu_erf":
        y = torch.nn.functional.gelu(y)
    elif epilogue == "residual":
        y = residual.double() + y
    return y


GEMM_SHAPES = [(1, 64, 64), (7, 200, 96), (33, 777, 144), (130, 50, 320), (64, 1000, 96), (257, 130, 72)]


# beside those: each width of the row-wise kernel (4, 8 and 16 features a workgroup), chunks of K
# with a tail, more chunks than waves, a K that is no multiple of 4 (the one-thread-an-element form)
F32_SHAPES = GEMM_SHAPES + [(16, 1500, 100), (9, 2600, 260), (5, 3000, 72), (12, 40, 6), (40, 2561, 132), (3, 1024, 1028),
                            (16, 33, 3076), (20, 70, 50),
                            # 17 to 64 rows in one workgroup: 16 features a workgroup with 2, 3 and 4 rows a thread,
                            # 8 with 1 and 2, 4 with a long K
                            (24, 4100, 200), (45, 4097, 68), (64, 4800, 324), (30, 2050, 1604), (17, 100, 3076),
                            # large enough for the tiles of 128 x 128 (528 of them), with edges on both sides and a K that ends inside a step of 16
                            (1100, 7300, 68)]


@pytest.mark.parametrize("epilogue", ["none", "gelu_tanh", "gelu_erf", "residual"])
@pytest.mark.parametrize("M,N,K", F32_SHAPES)
def test_gemm_float32(ops, M, N, K, epilogue):
    a, w, bias = rnd(M, K), rnd(N, K, seed=1, scale=0.2), rnd(N, seed=2)
    if epilogue == "residual":
        res = rnd(M, N, seed=3)
        want = gemm_reference(a, w, bias, epilogue, res)
        ops.gemm(a, w, bias, residual=res, epilogue=ops.EPI_RESIDUAL)
        close(res, want, 2e-6, "gemm f32 residual")
    else:
        out = torch.empty(M, N, device=DEV)
        ops.gemm(a, w, bias, out=out, epilogue=ops.ACTIVATION_EPILOGUE[epilogue])
        close(out, gemm_reference(a, w, bias, epilogue), 2e-6, f"gemm f32 {epilogue}")
    # a row's result does not depend on the rows around it, nor on which kernel their number chooses
    if M > 1:
        one = torch.empty(1, N, device=DEV)
        ops.gemm(a[M // 2:M // 2 + 1], w, bias, out=one)
        full = torch.empty(M, N, device=DEV)
        ops.gemm(a, w, bias, out=full)
        assert torch.equal(one[0], full[M // 2])
        many = torch.empty(70 + M, N, device=DEV)  # among 70 rows more: the tiled kernel, or the row-wise one again
        rows = torch.cat([rnd(70, K, seed=9), a])
        ops.gemm(rows, w, bias, out=many)
        assert torch.equal(many[70:], full)
        # from an address that is no multiple of 16 bytes the tiled kernel takes more than 64 rows, however few its tiles
        shifted = torch.empty(rows.numel() + 1, device=DEV)[1:].view_as(rows).copy_(rows)
        assert shifted.data_ptr() % 16 != 0
        ops.gemm(shifted, w, bias, out=many)
        assert torch.equal(many[70:], full)


@pytest.mark.parametrize("kernel", ["simple", "mfma128", "mfma64", "mfma128x64", "auto", "skinny1", "skinny4", "skinny16", "skinny4w", "skinny2w", "skinny8m1", "skinny4m2", "skinny2m4",
                                    "dl2", "dl6", "dl8", "dl15", "dl16", "dl17"])
@pytest.mark.parametrize("epilogue", ["none", "gelu_tanh", "gelu_erf", "residual"])
@pytest.mark.parametrize("M,N,K", GEMM_SHAPES + [(300, 264, 1600), (2, 50257 // 16, 64), (8, 130, 3072), (16, 2304, 768), (3, 40, 200), (17, 100, 64), (40, 333, 768), (64, 257, 1600),
                                                 (500, 300, 128), (129, 193, 192), (20, 4800, 1600), (600, 520, 256), (1030, 770, 128), (5, 100, 16384)])
def test_gemm_bfloat16(ops, M, N, K, epilogue, kernel):
    a, w, bias = rnd(M, K, dtype=torch.bfloat16), rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16), rnd(N, seed=2)
    tiles = {"mfma128": 1, "mfma64": 2, "mfma128x64": 3}

    if kernel.startswith("skinny") and M > 64:
        pytest.skip("the skinny kernel takes at most 64 rows")

    if kernel.startswith("dl") and K % 64 != 0:
        pytest.skip("the direct-load kernel takes K in multiples of 64")

    def run(**kw):
        if kernel.startswith("dl"):
            ops.gemm_mfma_dl(a, w, bias, tile=int(kernel[2:]), **kw)
        elif kernel.startswith("skinny"):
            spec, _, mtile = kernel[6:].partition("m")  # split of K, "w" for wide tiles of N, "m<tiles of rows>"
            ops.gemm_skinny(a, w, bias, ksplit=int(spec.rstrip("w")), wide=1 if spec.endswith("w") else 0,
                            mtile=int(mtile or 0), **kw)
        elif kernel == "simple":
            ops.gemm_simple(a, w, bias, **kw)
        elif kernel == "auto":
            ops.gemm(a, w, bias, **kw)
        else:
            ops.gemm_mfma(a, w, bias, tile=tiles[kernel], **kw)

    if epilogue == "residual":
        res = rnd(M, N, seed=3)
        want = gemm_reference(a, w, bias, epilogue, res)
        run(residual=res, epilogue=ops.EPI_RESIDUAL)
        close(res, want, 1e-5, f"gemm bf16 residual {kernel}")
    else:
        for out_dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 5e-3)):
            out = torch.empty(M, N, dtype=out_dtype, device=DEV)
            run(out=out, epilogue=ops.ACTIVATION_EPILOGUE[epilogue])
            close(out, gemm_reference(a, w, bias, epilogue), tol, f"gemm bf16 {epilogue} {kernel} -> {out_dtype}")


@pytest.mark.parametrize("epilogue", ["none", "gelu_tanh", "gelu_erf"])
@pytest.mark.parametrize("M,N,K,eps,parts", [(1, 64, 64, 1e-5, 1), (8, 2304, 768, 1e-5, 4), (16, 100, 1600, 1e-6, 2), (5, 777, 144, 1e-5, 3),
                                             (3, 50, 2048, 1e-3, 5), (13, 520, 1024, 1e-5, 1), (9, 3072, 768, 1e-5, 2), (16, 48, 96, 1e-6, 16),
                                             (17, 200, 768, 1e-5, 2), (32, 2304, 768, 1e-5, 1), (24, 130, 1600, 1e-6, 3), (29, 3072, 768, 1e-5, 1),
                                             (32, 90, 1024, 1e-5, 4)])
def test_gemm_with_layernorm_folded_in(ops, M, N, K, eps, parts, epilogue):
    """The product kernel that normalises its own rows, given whole or as a sum of planes: the
    same bits as the standalone norm followed by the streaming product."""
    planes = rnd(parts, M, K, scale=2.0)
    planes[0] += 0.5
    lw, lb = rnd(K, seed=5) + 1.0, rnd(K, seed=6)
    w, bias = rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16), rnd(N, seed=2)
    x = planes if parts > 1 else planes[0]
    h = torch.nn.functional.layer_norm(planes.double().sum(0), (K,), lw.double(), lb.double(), eps).to(torch.bfloat16)
    epi = ops.ACTIVATION_EPILOGUE[epilogue]
    for out_dtype in (torch.float32, torch.bfloat16):
        out = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
        ops.gemm_skinny_ln(x, lw, lb, eps, w, bias, out=out, epilogue=epi, wide=0)
        if M <= 16:
            strips_of_32 = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
            ops.gemm_skinny_ln(x, lw, lb, eps, w, bias, out=strips_of_32, epilogue=epi, wide=1)
            assert torch.equal(out, strips_of_32)
        # the folded norm rounds to bfloat16 where the standalone kernel does: allow one ulp of the operand
        close(out, gemm_reference(h, w, bias, epilogue), 4e-3 if out_dtype == torch.float32 else 8e-3, f"gemm+ln {epilogue}")
        normed = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
        ops.layernorm(normed, x, lw, lb, eps)
        two = torch.empty(M, N, dtype=out_dtype, device=DEV)
        ops.gemm_skinny(normed, w, bias, out=two, epilogue=epi, ksplit=8, wide=0, mtile=1 if M <= 16 else 0)
        if M <= 16:
            assert torch.equal(out, two)
        else:  # more tiles of rows: the plain kernel deals K out to its waves in another order
            close(out, two, 1e-5 if out_dtype == torch.float32 else 8e-3, "folded against norm + product")
    with pytest.raises(Exception, match="residual"):
        ops.gemm_skinny_ln(x, lw, lb, eps, w, bias, out=out, epilogue=ops.EPI_RESIDUAL)
    with pytest.raises(Exception, match="outside"):
        ops.gemm_skinny_ln(rnd(33, K), lw, lb, eps, w, bias, out=torch.empty(33, N, device=DEV))


def test_gemm_strided_rows_and_refusals(ops):
    from liyab_amd import KernelError

    wide = rnd(20, 256, dtype=torch.bfloat16)
    a = wide[:, 64:128]  # a view into a wider buffer: rows strided
    w = rnd(48, 64, dtype=torch.bfloat16, seed=1)
    out = torch.empty(20, 48, device=DEV)
    ops.gemm(a, w, None, out=out)
    close(out, a.double() @ w.double().t(), 1e-5, "strided a")
    with pytest.raises(KernelError):
        ops.gemm(a, rnd(48, 63, dtype=torch.bfloat16), None, out=out)  # K mismatch
    with pytest.raises(KernelError):
        ops.gemm(a, w, rnd(47), out=out)  # bias length
    with pytest.raises(KernelError):
        ops.gemm(a.float(), w, None, out=out)  # mixed dtypes
    with pytest.raises(KernelError):
        ops.gemm_mfma(rnd(4, 20, dtype=torch.bfloat16), rnd(8, 20, dtype=torch.bfloat16), None, out=torch.empty(4, 8, device=DEV))  # K % 8
    with pytest.raises(KernelError):
        ops.gemm(a, w, None, out=torch.empty(20, 48))  # not on the GPU


# ---------------------------------------------------------------------------
# attention over pages
# ---------------------------------------------------------------------------
def paged_case(n_seqs, ctx_lens, q_lens, H, Hkv, hd, page, dtype, seed=0, shuffle=True):
    """Random requests in a shuffled page pool; returns everything the kernels take and a
    float64 reference per token."""
    g = torch.Generator().manual_seed(seed)
    n_pages_per = [-(-c // page) for c in ctx_lens]
    total_pages = sum(n_pages_per) + 3
    perm = torch.randperm(total_pages, generator=g).tolist() if shuffle else list(range(total_pages))
    kc = torch.full((total_pages, Hkv, page, hd), float("nan"), dtype=dtype)
    vc = torch.full((total_pages, Hkv, page, hd), float("nan"), dtype=dtype)
    W = max(n_pages_per) + 1
    bt = torch.full((n_seqs, W), -1, dtype=torch.int32)
    ks, vs = [], []
    nxt = 0
    for s in range(n_seqs):
        k = (torch.randn(ctx_lens[s], Hkv, hd, generator=g)).to(dtype)
        v = (torch.randn(ctx_lens[s], Hkv, hd, generator=g)).to(dtype)
        ks.append(k)
        vs.append(v)
        for lp in range(n_pages_per[s]):
            pg = perm[nxt]
            nxt += 1
            bt[s, lp] = pg
            a, b = lp * page, min((lp + 1) * page, ctx_lens[s])
            kc[pg, :, :b - a] = k[a:b].transpose(0, 1)
            vc[pg, :, :b - a] = v[a:b].transpose(0, 1)
    tok_seq, tok_pos = [], []
    for s in range(n_seqs):
        for i in range(q_lens[s]):
            tok_seq.append(s)
            tok_pos.append(ctx_lens[s] - q_lens[s] + i)
    n = len(tok_seq)
    q = torch.randn(n, H * hd + 16, generator=g).to(dtype)  # wider than the heads: a strided view
    return dict(q=q, kc=kc, vc=vc, bt=bt, tok_seq=tok_seq, tok_pos=tok_pos, ks=ks, vs=vs, n=n)


def attention_reference(case, H, Hkv, hd, scale, window=0):
    out = torch.zeros(case["n"], H * hd, dtype=torch.float64)
    for t, (s, p) in enumerate(zip(case["tok_seq"], case["tok_pos"])):
        first = max(0, p - window + 1) if window > 0 else 0
        for h in range(H):
            hk = h // (H // Hkv)
            qv = case["q"][t, h * hd:(h + 1) * hd].double()
            k = case["ks"][s][first:p + 1, hk].double()
            v = case["vs"][s][first:p + 1, hk].double()
            w = torch.softmax((k @ qv) * scale, dim=0)
            out[t, h * hd:(h + 1) * hd] = w @ v
    return out


def run_attention(ops, case, H, hd, scale, window, kernel, splits=1, tok_list=None, waves=4, ksplit=1):
    dev = lambda x: x.to(DEV)  # noqa: E731
    q, kc, vc, bt = dev(case["q"]), dev(case["kc"]), dev(case["vc"]), dev(case["bt"])
    tok_seq = torch.tensor(case["tok_seq"], dtype=torch.int32, device=DEV)
    tok_pos = torch.tensor(case["tok_pos"], dtype=torch.int32, device=DEV)
    out = torch.zeros(case["n"], H * hd, dtype=q.dtype, device=DEV)
    qv = q[:, :H * hd]
    if kernel == "generic":
        ops.attention_generic(out, qv, kc, vc, bt, tok_seq, tok_pos, n_head=H, scale=scale, window=window)
    elif kernel == "prefill":
        work, row = [], 0
        lens = {}
        for sidx in case["tok_seq"]:
            lens[sidx] = lens.get(sidx, 0) + 1
        tile = splits if splits in (64, 128) else 128
        for sidx, nq in sorted(lens.items()):
            p0 = case["tok_pos"][row]
            for t0 in range(0, nq, tile):
                work.extend((sidx, row + t0, p0 + t0, min(tile, nq - t0)))
            row += nq
        wk = torch.tensor(work, dtype=torch.int32, device=DEV)
        ops.attention_prefill(out, qv, kc, vc, bt, wk, len(work) // 4, n_head=H, scale=scale, window=window, tile=tile,
                              ksplit=ksplit)
    elif kernel == "decode":
        partials = torch.empty(case["n"] * H * splits * (hd + 4), device=DEV) if splits > 1 else None
        tl = torch.tensor(tok_list, dtype=torch.int32, device=DEV) if tok_list is not None else None
        ops.attention_decode(out, qv, kc, vc, bt, tok_seq, tok_pos, n_head=H, scale=scale, window=window,
                             n_splits=splits, partials=partials, tok_list=tl, waves=waves,
                             n_tokens=len(tok_list) if tok_list is not None else None)
    return out


ATT_CASES = [
    # ctx_lens, q_lens, H, Hkv, hd, page
    ([1, 17, 300], [1, 1, 1], 4, 4, 16, 16),
    ([40, 129, 5], [7, 1, 5], 3, 3, 32, 16),
    ([700, 64], [1, 64], 5, 5, 64, 64),
    ([33, 257], [2, 3], 6, 2, 48, 8),
    ([100], [100], 2, 1, 128, 16),
    ([90, 31], [1, 1], 2, 2, 256, 16),
    ([50, 3], [4, 3], 3, 3, 80, 4),
    ([300, 40, 90], [8, 8, 8], 4, 2, 64, 16),
    # pages that are no power of two: page and offset by division
    ([130, 24, 49], [3, 1, 8], 3, 3, 32, 24),
    ([200, 97], [1, 5], 4, 2, 64, 48),
]


@pytest.mark.parametrize("window", [0, 37])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case_id", range(len(ATT_CASES)))
def test_attention_generic(ops, case_id, dtype, window):
    ctx_lens, q_lens, H, Hkv, hd, page = ATT_CASES[case_id]
    case = paged_case(len(ctx_lens), ctx_lens, q_lens, H, Hkv, hd, page, dtype, seed=case_id)
    scale = 0.7 / math.sqrt(hd)
    out = run_attention(ops, case, H, hd, scale, window, "generic")
    close(out, attention_reference(case, H, Hkv, hd, scale, window), 2e-6 if dtype == torch.float32 else 8e-3, "generic")


@pytest.mark.parametrize("window", [0, 37])
@pytest.mark.parametrize("splits,waves", [(1, 4), (1, 16), (2, 4), (5, 16), (32, 4), (1, 8), (3, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case_id", range(len(ATT_CASES)))
def test_attention_decode(ops, case_id, dtype, splits, waves, window):
    ctx_lens, q_lens, H, Hkv, hd, page = ATT_CASES[case_id]
    case = paged_case(len(ctx_lens), ctx_lens, q_lens, H, Hkv, hd, page, dtype, seed=case_id)
    scale = 0.7 / math.sqrt(hd)
    out = run_attention(ops, case, H, hd, scale, window, "decode", splits, waves=waves)
    assert torch.isfinite(out.float()).all()
    close(out, attention_reference(case, H, Hkv, hd, scale, window), 8e-3 if dtype == torch.bfloat16 else 2e-6, f"decode splits={splits}")
    # a subset of the rows through tok_list: the others stay untouched
    if case["n"] > 2:
        rows = list(range(case["n"]))[::2]
        part = run_attention(ops, case, H, hd, scale, window, "decode", splits, tok_list=rows, waves=waves)
        assert torch.equal(part[rows], out[rows]) and (part[1::2] == 0).all()


@pytest.mark.parametrize("window", [0, 37, 300])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case_id", range(len(ATT_CASES)))
def test_attention_splits_by_position(ops, case_id, dtype, window):
    """Splits of a fixed number of keys from a token's first key on: right against the plain
    formula, and the same bits whether the step has just the splits the longest context needs or
    more (a longer context beside it), the later ones empty; a context within one split has the
    bits of the unsplit call."""
    ctx_lens, q_lens, H, Hkv, hd, page = ATT_CASES[case_id]
    case = paged_case(len(ctx_lens), ctx_lens, q_lens, H, Hkv, hd, page, dtype, seed=case_id)
    scale = 0.7 / math.sqrt(hd)
    dev = lambda x: x.to(DEV)  # noqa: E731
    q, kc, vc, bt = dev(case["q"]), dev(case["kc"]), dev(case["vc"]), dev(case["bt"])
    tok_seq = torch.tensor(case["tok_seq"], dtype=torch.int32, device=DEV)
    tok_pos = torch.tensor(case["tok_pos"], dtype=torch.int32, device=DEV)
    chunk = 64
    longest = max(ctx_lens) if window == 0 else min(max(ctx_lens), window)
    need = -(-longest // chunk)
    outs = []
    for splits in (need, need + 1, 2 * need + 3):
        out = torch.zeros(case["n"], H * hd, dtype=dtype, device=DEV)
        partials = torch.full((case["n"] * H * splits * (hd + 4),), float("nan"), device=DEV) if splits > 1 else None
        ops.attention_decode(out, q[:, :H * hd], kc, vc, bt, tok_seq, tok_pos, n_head=H, scale=scale, window=window,
                             n_splits=splits, partials=partials, waves=4, chunk=chunk)
        assert torch.isfinite(out.float()).all()
        outs.append(out)
    close(outs[0], attention_reference(case, H, Hkv, hd, scale, window), 8e-3 if dtype == torch.bfloat16 else 2e-6, "splits by position")
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    # launched as one split, a workgroup walking its token's splits in turn: the same bits again
    if need <= 16:
        out = torch.zeros(case["n"], H * hd, dtype=dtype, device=DEV)
        ops.attention_decode(out, q[:, :H * hd], kc, vc, bt, tok_seq, tok_pos, n_head=H, scale=scale, window=window,
                             n_splits=1, waves=4, chunk=chunk)
        assert torch.equal(out, outs[0]), "one workgroup walking the splits"
    # each request alone, with the splits its own context needs
    for s_, n_ctx in enumerate(ctx_lens):
        rows = [t for t, r in enumerate(case["tok_seq"]) if r == s_]
        own = -(-(n_ctx if window == 0 else min(n_ctx, window)) // chunk)
        out = torch.zeros(case["n"], H * hd, dtype=dtype, device=DEV)
        partials = torch.empty(len(rows) * H * own * (hd + 4), device=DEV) if own > 1 else None
        ops.attention_decode(out, q[:, :H * hd], kc, vc, bt, tok_seq, tok_pos, n_head=H, scale=scale, window=window,
                             n_splits=own, partials=partials, waves=4, chunk=chunk,
                             tok_list=torch.tensor(rows, dtype=torch.int32, device=DEV), n_tokens=len(rows))
        assert torch.equal(out[rows], outs[0][rows]), f"request {s_} alone"


@pytest.mark.parametrize("waves", [4, 16])
@pytest.mark.parametrize("window", [0, 37])
@pytest.mark.parametrize("splits", [2, 4, 7, 8])
@pytest.mark.parametrize("case_id", [0, 1, 2, 3, 5, 6, 7, 8, 9])
def test_attention_splits_merged_by_the_projection(ops, case_id, splits, window, waves):
    """Attention that leaves each (token, head) pair's keys in splits, and the projection cut
    over its inner dimension that merges them as it loads them: the planes add up to rows +
    attention . W^T + bias; the merge kernel gives attention's output from the same splits.
    Contexts shorter than the number of splits leave splits empty."""
    ctx_lens, q_lens, H, Hkv, hd, page = ATT_CASES[case_id]
    case = paged_case(len(ctx_lens), ctx_lens, q_lens, H, Hkv, hd, page, torch.bfloat16, seed=case_id)
    scale = 0.7 / math.sqrt(hd)
    n = case["n"]
    dev = lambda x: x.to(DEV)  # noqa: E731
    q, kc, vc, bt = dev(case["q"]), dev(case["kc"]), dev(case["vc"]), dev(case["bt"])
    tok_seq = torch.tensor(case["tok_seq"], dtype=torch.int32, device=DEV)
    tok_pos = torch.tensor(case["tok_pos"], dtype=torch.int32, device=DEV)
    partials = torch.full((n, H, splits, hd + 4), float("nan"), device=DEV)
    untouched = torch.full((n, H * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.attention_decode(untouched, q[:, :H * hd], kc, vc, bt, tok_seq, tok_pos, n_head=H, scale=scale, window=window,
                         n_splits=splits, partials=partials, waves=waves, leave_splits=True)
    assert (untouched == 7.0).all()
    want = attention_reference(case, H, Hkv, hd, scale, window)
    merged = torch.empty(n, H * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention_merge(merged, partials)
    close(merged, want, 8e-3, "merged splits")
    N, K = 72, H * hd
    w, bias = rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16), rnd(N, seed=2)
    for parts in (1, 2, 3):
        if (parts - 1) * (((K + 63) // 64 + parts - 1) // parts) >= (K + 63) // 64:
            continue
        for n_base in (None, 0, 2):
            base = None if n_base is None else (rnd(n, N, seed=8, scale=3.0) if n_base == 0 else rnd(n_base, n, N, seed=9, scale=3.0))
            planes = torch.full((parts, n, N), float("nan"), device=DEV)
            if n > 32:
                with pytest.raises(Exception, match="outside"):
                    ops.gemm_att_parts(partials, w, planes, bias=bias if base is not None else None, base=base)
                continue
            ops.gemm_att_parts(partials, w, planes, bias=bias if base is not None else None, base=base)
            total = merged.double() @ w.double().t()
            if base is not None:
                total = total + bias.double() + (base.double() if n_base == 0 else base.double().sum(0))
            close(planes.double().sum(0), total, 1e-5, f"projection over splits, {parts} parts, base {n_base}")
            # the same bits as the plain cut product over the merged rows
            two = torch.empty_like(planes)
            ops.gemm_skinny_parts(merged, w, two, bias=bias if base is not None else None, base=base, ksplit=8)
            assert torch.equal(planes, two)


def test_projection_over_splits_with_rows_32_kb_apart(ops):
    """Heads x head size = 16,384: the weights' rows lie 32 KB apart, where the streaming kernels
    walk K in blocks from a place of each workgroup's own; the kernel that merges attention's
    splits as it loads them must still give the bits of the merge followed by the plain product."""
    M, H, S, hd, N = 3, 128, 2, 128, 40
    g = torch.Generator().manual_seed(3)
    partials = torch.randn(M, H, S, hd + 4, generator=g)
    partials[..., hd] = torch.randn(M, H, S, generator=g) * 2  # the splits' maxima
    partials[..., hd + 1] = torch.rand(M, H, S, generator=g) * 50 + 1  # and sums
    partials = partials.to(DEV)
    merged = torch.empty(M, H * hd, dtype=torch.bfloat16, device=DEV)
    ops.attention_merge(merged, partials)
    w, bias = rnd(N, H * hd, seed=1, scale=0.05, dtype=torch.bfloat16), rnd(N, seed=2)
    base = rnd(M, N, seed=8, scale=3.0)
    with pytest.raises(Exception, match="do not fit LDS"):  # whole rows of 16,384 are refused, not mangled
        ops.gemm_att_parts(partials, w, torch.empty(1, M, N, device=DEV), bias=bias, base=base)
    for parts in (2, 4):
        planes = torch.full((parts, M, N), float("nan"), device=DEV)
        ops.gemm_att_parts(partials, w, planes, bias=bias, base=base)
        want = merged.double() @ w.double().t() + bias.double() + base.double()
        close(planes.double().sum(0), want, 1e-5, f"projection over splits at K = 16,384, {parts} parts")
        two = torch.empty_like(planes)
        ops.gemm_skinny_parts(merged, w, two, bias=bias, base=base, ksplit=8)
        assert torch.equal(planes, two)


PREFILL_CASES = [
    # ctx_lens, q_lens, H, Hkv, hd, page
    ([1, 17, 300], [1, 17, 300], 4, 4, 16, 16),
    ([40, 129, 5], [7, 100, 5], 3, 3, 32, 16),
    ([700, 64], [130, 64], 5, 5, 64, 64),
    ([33, 257], [20, 129], 6, 2, 48, 8),
    ([300], [300], 2, 1, 128, 16),
    ([90, 31], [31, 9], 2, 2, 80, 16),
    ([1024], [1024], 1, 1, 64, 16),
    # pages that are no power of two
    ([130, 24, 49], [100, 24, 40], 3, 3, 32, 24),
    ([400, 97], [200, 97], 4, 2, 64, 48),
]


@pytest.mark.parametrize("tile,ksplit", [(64, 1), (64, 2), (64, 4), (128, 1), (128, 2)])
@pytest.mark.parametrize("window", [0, 37, 200])
@pytest.mark.parametrize("case_id", range(len(PREFILL_CASES)))
def test_attention_prefill(ops, case_id, window, tile, ksplit):
    ctx_lens, q_lens, H, Hkv, hd, page = PREFILL_CASES[case_id]
    if ksplit == 4 and hd > 64:
        pytest.skip("4 waves a query group are taken up to head size 64")
    case = paged_case(len(ctx_lens), ctx_lens, q_lens, H, Hkv, hd, page, torch.bfloat16, seed=case_id)
    scale = 0.7 / math.sqrt(hd)
    out = run_attention(ops, case, H, hd, scale, window, "prefill", splits=tile, ksplit=ksplit)
    assert torch.isfinite(out.float()).all()
    close(out, attention_reference(case, H, Hkv, hd, scale, window), 8e-3, "prefill")


def reference_from_pages(case, kc, vc, bt, H, Hkv, hd, page, scale, window=0):
    """The plain formula over whatever pages a block table names (float64)."""
    out = torch.zeros(case["n"], H * hd, dtype=torch.float64)
    for t, (s, p) in enumerate(zip(case["tok_seq"], case["tok_pos"])):
        first = max(0, p - window + 1) if window > 0 else 0
        pos = torch.arange(first, p + 1)
        pages, offs = bt[s, pos // page].long(), pos % page
        for h in range(H):
            hk = h // (H // Hkv)
            k, v = kc[pages, hk, offs].double(), vc[pages, hk, offs].double()
            w = torch.softmax((k @ case["q"][t, h * hd:(h + 1) * hd].double()) * scale, dim=0)
            out[t, h * hd:(h + 1) * hd] = w @ v
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("kernel", ["generic", "decode", "decode in splits", "prefill"])
def test_a_page_id_past_the_counted_pages_is_not_followed(ops, kernel, dtype):
    """The caches hold eight pages more than the launcher is told of, and block tables name ids
    in that slack (and a -1 in a place that is read): told the count, a kernel reads the last
    counted page instead; told of all pages it reads the slack page. Either way every fetch
    stays inside the caches: an id that a table should never hold costs a wrong number, not
    the machine."""
    if kernel == "prefill" and dtype != torch.bfloat16:
        pytest.skip("the tiled kernel is bfloat16 only")
    ctx_lens, q_lens, H, Hkv, hd, page = ([300, 70], [9, 40], 4, 2, 64, 16) if kernel == "prefill" else ([300, 70], [3, 1], 4, 2, 64, 16)
    case = paged_case(len(ctx_lens), ctx_lens, q_lens, H, Hkv, hd, page, dtype, seed=11)
    counted = case["kc"].shape[0]
    g = torch.Generator().manual_seed(5)
    kc = torch.cat([torch.nan_to_num(case["kc"].float(), nan=0.5), torch.randn(8, Hkv, page, hd, generator=g)]).to(dtype)
    vc = torch.cat([torch.nan_to_num(case["vc"].float(), nan=-0.5), torch.randn(8, Hkv, page, hd, generator=g)]).to(dtype)
    bt = case["bt"].clone()
    bt[0, 2], bt[0, 7], bt[1, 1] = counted + 3, counted + 7, -1
    case = dict(case, kc=kc, vc=vc, bt=bt)
    scale = 0.7 / math.sqrt(hd)
    tol = 8e-3 if dtype == torch.bfloat16 else 2e-6

    def run(num_pages):
        dev = lambda x: x.to(DEV)  # noqa: E731
        q = dev(case["q"])[:, :H * hd]
        tok_seq = torch.tensor(case["tok_seq"], dtype=torch.int32, device=DEV)
        tok_pos = torch.tensor(case["tok_pos"], dtype=torch.int32, device=DEV)
        out = torch.zeros(case["n"], H * hd, dtype=dtype, device=DEV)
        kw = dict(n_head=H, scale=scale, num_pages=num_pages)
        if kernel == "generic":
            ops.attention_generic(out, q, dev(kc), dev(vc), dev(bt), tok_seq, tok_pos, **kw)
        elif kernel == "prefill":
            work = torch.tensor([0, 0, ctx_lens[0] - q_lens[0], q_lens[0], 1, q_lens[0], ctx_lens[1] - q_lens[1], q_lens[1]],
                                dtype=torch.int32, device=DEV)
            ops.attention_prefill(out, q, dev(kc), dev(vc), dev(bt), work, 2, tile=64, **kw)
        else:
            splits = 3 if kernel == "decode in splits" else 1
            partials = torch.empty(case["n"] * H * splits * (hd + 4), device=DEV) if splits > 1 else None
            ops.attention_decode(out, q, dev(kc), dev(vc), dev(bt), tok_seq, tok_pos, n_splits=splits, partials=partials, **kw)
        assert torch.isfinite(out.float()).all()
        return out

    told = run(counted)
    close(told, reference_from_pages(case, kc, vc, bt.clamp(0, counted - 1), H, Hkv, hd, page, scale), tol, "ids brought into the counted pages")
    whole = run(None)
    close(whole, reference_from_pages(case, kc, vc, bt.clamp(0, counted + 7), H, Hkv, hd, page, scale), tol, "every page counted")
    assert not torch.equal(told, whole)
    with pytest.raises(Exception, match="pages"):
        run(counted + 9)


@pytest.mark.parametrize("kernel", ["kv_write", "skinny", "dl", "mfma", "folded norm"])
def test_a_slot_past_the_counted_pages_is_not_written(ops, kernel):
    """Slots in the eight pages the launcher is not told of (and a -1) are skipped; told of all
    pages, the same call writes them."""
    M, H, Hkv, hd, K, page = 24, 3, 3, 32, 128, 8
    q_dim, kv_dim = H * hd, Hkv * hd
    N = q_dim + 2 * kv_dim
    counted = 6
    a, w, bias = rnd(M, K, dtype=torch.bfloat16), rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16), rnd(N, seed=2)
    slots = torch.randperm(counted * page)[:M].to(torch.int32)
    slots[3], slots[10], slots[17] = counted * page, (counted + 8) * page - 1, -1
    slots = slots.to(DEV)

    def run(num_pages):
        kc = torch.zeros(counted + 8, Hkv, page, hd, dtype=torch.bfloat16, device=DEV)
        vc = torch.zeros_like(kc)
        q = torch.zeros(M, q_dim, dtype=torch.bfloat16, device=DEV)
        kw = dict(out=q, epilogue=ops.EPI_QKV_PAGED, kv=(kc, vc, slots, q_dim, num_pages))
        if kernel == "kv_write":
            full = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            ops.gemm_simple(a, w, bias, out=full)
            ops.kv_write(kc, vc, full, q_dim, q_dim + kv_dim, slots, num_pages=num_pages)
        elif kernel == "skinny":
            ops.gemm_skinny(a, w, bias, **kw)
        elif kernel == "dl":
            ops.gemm_mfma_dl(a, w, bias, tile=2, **kw)
        elif kernel == "mfma":
            ops.gemm_mfma(a, w, bias, tile=2, **kw)
        else:
            x = rnd(M, K, scale=2.0, seed=4)
            ops.gemm_skinny_ln(x, rnd(K, seed=5) + 1.0, rnd(K, seed=6), 1e-5, w, bias, **kw)
        return kc, vc

    for num_pages, written in ((counted, M - 3), (None, M - 1)):
        kc, vc = run(num_pages)
        for c in (kc, vc):
            assert (c[:counted] != 0).any(dim=(1, 3)).sum().item() == M - 3  # the tokens with a slot in the counted pages
            assert (c != 0).any(dim=(1, 3)).sum().item() == written


@pytest.mark.parametrize("T,targets", [(700, [0, 15, 16, 31, 32, 255, 256, 511, 559, 560, 561, 600, 640, 687, 698, 699]),
                                       (5000, [0, 17, 1023, 1024, 2047, 2048, 3000, 4095, 4096, 4097, 4859, 4860, 4900, 4959, 4998, 4999])])
def test_attention_prefill_finds_one_far_key(ops, T, targets):
    """A portion's queries each with one outstanding key, at page and block edges; in a context of
    700 positions and in one of 5,000 (313 pages)."""
    H = Hkv = 2
    hd, page, nq = 64, 16, 140
    case = paged_case(1, [T], [nq], H, Hkv, hd, page, torch.bfloat16, seed=3)
    k = case["ks"][0]
    for n, target in enumerate(targets):
        row = nq - 1 - n * 3  # the query at position T - 1 - 3 n looks for `target` if it may see it
        qpos = T - nq + row
        if target > qpos:
            continue
        qv = case["q"][row, :hd].float()
        # orthogonalise against earlier planted keys is not needed: random 64-vectors are nearly orthogonal
        k[target, 0] = (qv * 4).to(torch.bfloat16)
        lp, off = divmod(target, page)
        case["kc"][case["bt"][0, lp], 0, off] = k[target, 0]
    out = run_attention(ops, case, H, hd, 1.0, 0, "prefill")
    ref = attention_reference(case, H, Hkv, hd, 1.0, 0)
    close(out, ref, 8e-3, "prefill far keys")


@pytest.mark.parametrize("T,targets", [(700, (0, 15, 16, 17, 255, 256, 511, 512, 687, 688, 698, 699)),
                                       (5000, (0, 255, 256, 2047, 2048, 4095, 4096, 4863, 4864, 4998, 4999))])
@pytest.mark.parametrize("kernel", ["generic", "decode", "decode by position", "decode walking its splits"])
def test_attention_finds_one_far_key(ops, kernel, T, targets):
    """Random values average a wrong key away; here one key's score stands out, at a page's
    first and last slot, in the first page and the last, at the edges of splits, and the output
    must be its value row; in a context of 700 positions and in one of 5,000."""
    H = Hkv = 2
    hd, page = 64, 16
    if kernel == "decode walking its splits" and T > 16 * 256:
        pytest.skip("one workgroup walks at most 16 splits")
    for target in targets:
        case = paged_case(1, [T], [1], H, Hkv, hd, page, torch.bfloat16, seed=target)
        qv = case["q"][0, :hd].float()
        k = case["ks"][0]
        k[target, 0] = (qv * 4).to(torch.bfloat16)  # head 0: score ~ 4 |q|^2 ~ 250, all others ~ N(0, 8)
        lp, off = divmod(target, page)
        case["kc"][case["bt"][0, lp], 0, off] = k[target, 0]
        if kernel.startswith("decode "):
            dev = lambda x: x.to(DEV)  # noqa: E731
            splits = -(-T // 256) if kernel == "decode by position" else 1
            out = torch.zeros(1, H * hd, dtype=torch.bfloat16, device=DEV)
            ops.attention_decode(out, dev(case["q"])[:, :H * hd], dev(case["kc"]), dev(case["vc"]), dev(case["bt"]),
                                 torch.zeros(1, dtype=torch.int32, device=DEV), torch.tensor([T - 1], dtype=torch.int32, device=DEV),
                                 n_head=H, scale=1.0, n_splits=splits, waves=4, chunk=256,
                                 partials=torch.empty(H * splits * (hd + 4), device=DEV) if splits > 1 else None)
        else:
            out = run_attention(ops, case, H, hd, 1.0, 0, kernel, splits=(3 if T < 1000 else 11) if kernel == "decode" else 1)
        want = case["vs"][0][target, 0].float()
        assert torch.allclose(out[0, :hd].float().cpu(), want, atol=2e-2), f"{kernel}: key {target} was not found"


# ---------------------------------------------------------------------------
# sampling
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("rows,V", [(1, 50257), (9, 1000), (64, 777), (3, 5)])
def test_argmax_ties_go_to_the_lowest_id(ops, rows, V):
    logits = rnd(rows, V + 3)[:, :V]  # strided rows
    logits[:, V // 2] = 50.0
    logits[:, V - 1] = 50.0  # a tie: the lower id wins
    if rows > 1:
        logits[1, 0] = 50.0
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    ops.argmax(out, logits)
    want = [V // 2] * rows
    if rows > 1:
        want[1] = 0
    assert out.tolist() == want
    ops.argmax(out, rnd(rows, V, seed=4))
    assert out.tolist() == rnd(rows, V, seed=4).argmax(dim=1).tolist()


@pytest.mark.parametrize("V", [1000, 50257, 53250, 60000, 70001])
def test_sampler_against_the_plain_sampler(ops, V):
    """Temperature, top-k and top-p per row against the plain implementation's rules, at
    vocabularies that take each of the sampling kernels (the row in registers with a one-wave
    finish for top-k <= 64, the same with many candidates, and the general kernel)."""
    import plain_gpt2 as plain

    logits = rnd(14, V, scale=2.0, seed=11)
    logits[5, 100:140] = 3.0  # many ties at the top-k boundary
    logits[12, :] = 0.25  # all equal: ties everywhere
    logits[3, 7:60:2] = 9.0  # ties above the top-k boundary: all kept
    logits[4, 10:50] = 8.0  # ties at the top: the 5 of the lowest ids are kept
    logits[13, 300:900] = 7.5  # more ties at the boundary than keys the one-wave pool would hold at the large vocabularies
    params = [(0.0, 0, 1.0), (1.0, 0, 1.0), (0.8, 0, 1.0), (0.8, 40, 0.95), (1.3, 5, 1.0), (0.7, 20, 1.0), (1.0, 0, 0.5),
              (1.0, 0, 0.05), (0.5, 1, 1.0), (2.0, 999, 0.9), (1.0, 40, 0.0), (0.8, 0, 0.999), (1.0, 64, 0.7), (0.9, 65, 0.9)]
    cpu = logits.cpu().numpy()
    for trial in range(6):
        u = [plain.uniform(7 + trial, r) for r in range(len(params))]
        out = torch.empty(len(params), dtype=torch.int32, device=DEV)
        ops.sample(out, logits,
                   torch.tensor([p[0] for p in params], dtype=torch.float32, device=DEV),
                   torch.tensor([p[1] for p in params], dtype=torch.int32, device=DEV),
                   torch.tensor([p[2] for p in params], dtype=torch.float32, device=DEV),
                   torch.tensor(u, dtype=torch.float64, device=DEV))
        got = out.tolist()
        for r, (T, k, p) in enumerate(params):
            probs = plain.probabilities(cpu[r], T, k, p)
            want = plain.sample(probs, u[r])
            if got[r] != want:
                cdf = np.cumsum(probs)
                assert probs[got[r]] > 0 and np.abs(cdf - u[r]).min() < 1e-5, (V, r, params[r], got[r], want)


@pytest.mark.parametrize("V", [3000, 50257, 53250, 65533])
def test_top_p_over_many_candidates_keeps_exactly_the_nucleus(ops, V):
    """Top-p alone (and with a top-k too wide for one wave) at rows made so that a wrong cut shows
    in the draws: a few heavy ids over a light floor, the cut falling between them, inside a run
    of ties (the lowest ids of the run are kept), on the top-k boundary's ties, in a flat row where
    every key shares a bin, and in a peaked row whose masses span every bin. 48 draws a row are
    compared with the plain sampler's; a draw may differ only where the uniform number lies
    within rounding of a boundary between two ids."""
    import plain_gpt2 as plain

    g = torch.Generator().manual_seed(V)
    cases = []  # (logits row, temperature, top_k, top_p)
    floor = torch.randn(V, generator=g) * 0.5 - 12.0
    heavy = floor.clone()
    heavy[[5, 900, 1777, 2500, 40, 41]] = torch.tensor([3.0, 2.9, 2.5, 2.45, 1.0, 0.9])
    for p in (0.2, 0.4, 0.63, 0.8, 0.97, 0.99999):
        cases.append((heavy, 1.0, 0, p))
    ties = floor.clone()
    ties[[10, 20, 30]] = 6.0
    ties[100:2100:250] = 5.0  # eight ties: the cut falls among them
    for p in (0.3, 0.5, 0.7, 0.85, 0.95):
        cases.append((ties, 1.0, 0, p))
    cases.append((ties, 0.5, 0, 0.9))
    wide = torch.randn(V, generator=g) * 2.0
    wide[200:330] = 4.0  # 130 ties on the boundary of top-k 100: 100 - (keys above) of them are in the set
    for k, p in ((100, 0.5), (100, 0.9), (100, 0.999), (400, 0.3), (V - 1, 0.6)):
        cases.append((wide, 1.0, k, p))
    cases.append((torch.full((V,), 0.25), 1.0, 0, 0.5))  # every key in one bin: more than the pool holds
    zeros = (torch.randn(V, generator=g) * 1.5).round()  # thousands of ties a value, and both zeros, which are one value
    assert (zeros == 0).sum() > 100 and torch.signbit(zeros[zeros == 0]).any() and not torch.signbit(zeros[zeros == 0]).all()
    for T, k, p in ((1.0, 0, 0.6), (1.7, 0, 0.95), (1.0, 200, 0.9), (0.0, 0, 1.0), (1.0, 30, 1.0)):
        cases.append((zeros.clamp(max=0.0) if T == 0.0 else zeros, T, k, p))
    cases.append((torch.randn(V, generator=g) * 0.01, 1.0, 0, 0.9))  # nearly flat: a few bins hold the row
    peaked = torch.linspace(0.0, -40.0, V)[torch.randperm(V, generator=g)]
    for T, p in ((1.0, 0.9), (0.3, 0.5), (3.0, 0.95)):
        cases.append((peaked, T, 0, p))
    draws = 48
    for row, T, k, p in cases:
        logits = row.to(DEV).repeat(draws, 1)
        u = [plain.uniform(1000 + k, i) for i in range(draws)]
        u[0], u[1] = 0.0, 1.0 - 2.0 ** -40  # the first and the last id that are kept
        out = torch.empty(draws, dtype=torch.int32, device=DEV)
        ops.sample(out, logits, torch.full((draws,), T, dtype=torch.float32, device=DEV),
                   torch.full((draws,), k, dtype=torch.int32, device=DEV),
                   torch.full((draws,), p, dtype=torch.float32, device=DEV), torch.tensor(u, dtype=torch.float64, device=DEV))
        probs = plain.probabilities(row.numpy(), T, k, p)
        cdf = np.cumsum(probs)
        for i, got in enumerate(out.tolist()):
            want = plain.sample(probs, u[i])
            if got != want:
                assert probs[got] > 0 and np.abs(cdf - u[i]).min() < 1e-5, (V, T, k, p, i, got, want)


@pytest.mark.parametrize("V", [1000, 50257, 70001])
def test_sampler_without_cuts(ops, V):
    """Temperature alone, called without top-k and top-p: the shorter kernel draws what the
    plain sampler draws, also from a row of ties and beside a greedy row."""
    import plain_gpt2 as plain

    temps = [1.0, 0.8, 0.0, 1.7, 0.3, 1.0, 0.05]
    logits = rnd(len(temps), V, scale=2.0, seed=13)
    logits[5, :] = -1.5  # all equal
    logits[3, 40:90] = 6.0
    cpu = logits.cpu().numpy()
    with pytest.raises(ops.KernelError):
        ops.sample(torch.empty(len(temps), dtype=torch.int32, device=DEV), logits,
                   torch.tensor(temps, dtype=torch.float32, device=DEV), None,
                   torch.ones(len(temps), dtype=torch.float32, device=DEV),
                   torch.zeros(len(temps), dtype=torch.float64, device=DEV))
    for trial in range(8):
        u = [plain.uniform(23 + trial, r) for r in range(len(temps))]
        out = torch.empty(len(temps), dtype=torch.int32, device=DEV)
        ops.sample(out, logits, torch.tensor(temps, dtype=torch.float32, device=DEV), None, None,
                   torch.tensor(u, dtype=torch.float64, device=DEV))
        got = out.tolist()
        for r, T in enumerate(temps):
            probs = plain.probabilities(cpu[r], T, 0, 1.0)
            want = plain.sample(probs, u[r])
            if got[r] != want:
                cdf = np.cumsum(probs)
                assert probs[got[r]] > 0 and np.abs(cdf - u[r]).min() < 1e-5, (V, r, T, got[r], want)


@pytest.mark.parametrize("K", [64, 768, 832, 3072])
def test_tiles_of_every_shape_give_a_row_the_same_bits(ops, K):
    """The tiled products of the batch-invariant mode: the small tiles whose four groups of waves
    walk K side by side (16, 17) and the large ones whose one group keeps four sums by unit of K
    (102, 106, 108) leave the same bits in a row, whatever rows are beside it; K of one unit, of
    whole rounds of four units and of 13 units."""
    M, N = 200, 320
    a, w, bias = rnd(M, K, dtype=torch.bfloat16, seed=K), rnd(N, K, dtype=torch.bfloat16, seed=K + 1, scale=0.2), rnd(N, seed=2)
    want = gemm_reference(a.float(), w.float(), bias, "none")
    full = {}
    for tile in (102, 106, 108, 16, 17):
        out = torch.empty(M, N, device=DEV)
        ops.gemm_mfma_dl(a, w, bias, out=out, tile=tile)
        close(out, want, 2e-5, f"tile {tile}")
        full[tile] = out
    for tile in (106, 108, 16, 17):
        assert torch.equal(full[tile], full[102]), f"tile {tile} against 102"
    for rows in (slice(0, 8), slice(37, 38), slice(100, 164)):
        for tile in (16, 17):
            out = torch.empty(rows.stop - rows.start, N, device=DEV)
            ops.gemm_mfma_dl(a[rows], w, bias, out=out, tile=tile)
            assert torch.equal(out, full[108][rows]), f"rows {rows} in tiles {tile}"


@pytest.mark.parametrize("kernel", ["skinny", "mfma128", "mfma64", "dl2", "dl8", "dl15", "dl16", "auto"])
@pytest.mark.parametrize("M,H,Hkv,hd,K,page", [(5, 3, 3, 16, 64, 4), (40, 4, 2, 32, 128, 16), (200, 5, 5, 48, 192, 8), (130, 2, 1, 64, 64, 64), (700, 6, 3, 64, 128, 16),
                                               (50, 3, 3, 32, 128, 24), (300, 4, 2, 64, 192, 48)])
def test_gemm_paged_qkv_epilogue(ops, kernel, M, H, Hkv, hd, K, page):
    """Queries to a dense buffer, keys and values straight into shuffled cache slots, against
    the plain product followed by the scatter kernel."""
    if kernel == "skinny" and M > 64:
        pytest.skip("at most 64 rows")
    q_dim, kv_dim = H * hd, Hkv * hd
    N = q_dim + 2 * kv_dim
    a, w, bias = rnd(M, K, dtype=torch.bfloat16), rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16), rnd(N, seed=2)
    pages = -(-M // page) + 3
    slots = torch.randperm(pages * page)[:M].to(torch.int32).to(DEV)
    kc = torch.zeros(pages, Hkv, page, hd, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    q = torch.zeros(M, q_dim, dtype=torch.bfloat16, device=DEV)
    kw = dict(out=q, epilogue=ops.EPI_QKV_PAGED, kv=(kc, vc, slots, q_dim))
    if kernel == "skinny":
        ops.gemm_skinny(a, w, bias, **kw)
    elif kernel == "auto":
        ops.gemm(a, w, bias, **kw)
    elif kernel.startswith("dl"):
        ops.gemm_mfma_dl(a, w, bias, tile=int(kernel[2:]), **kw)
    else:
        ops.gemm_mfma(a, w, bias, tile=1 if kernel == "mfma128" else 2, **kw)
    full = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    ops.gemm_simple(a, w, bias, out=full)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    ops.kv_write(kc2, vc2, full, q_dim, q_dim + kv_dim, slots)
    close(q, full[:, :q_dim], 1e-2, "queries")
    close(kc, kc2, 1e-2, "keys")
    close(vc, vc2, 1e-2, "values")
    assert (kc == 0).sum() == (kc2 == 0).sum()  # nothing written outside the tokens' slots


@pytest.mark.parametrize("M,H,Hkv,hd,K,page", [(1, 4, 4, 16, 64, 16), (9, 6, 2, 32, 192, 8), (16, 12, 12, 64, 768, 64), (27, 5, 5, 48, 240, 16),
                                               (32, 12, 12, 64, 768, 64)])
def test_folded_norm_with_the_paged_qkv_epilogue(ops, M, H, Hkv, hd, K, page):
    """The product that normalises its own rows, writing queries to a dense buffer and keys and
    values into shuffled cache slots: what the standalone norm followed by the streaming
    product writes."""
    q_dim, kv_dim = H * hd, Hkv * hd
    N = q_dim + 2 * kv_dim
    x = rnd(2, M, K, scale=2.0)
    lw, lb = rnd(K, seed=5) + 1.0, rnd(K, seed=6)
    w, bias = rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16), rnd(N, seed=2)
    pages = -(-M // page) + 3
    slots = torch.randperm(pages * page)[:M].to(torch.int32).to(DEV)
    got = [torch.zeros(pages, Hkv, page, hd, dtype=torch.bfloat16, device=DEV) for _ in range(2)] + [torch.zeros(M, q_dim, dtype=torch.bfloat16, device=DEV)]
    ops.gemm_skinny_ln(x, lw, lb, 1e-5, w, bias, out=got[2], epilogue=ops.EPI_QKV_PAGED, kv=(got[0], got[1], slots, q_dim))
    normed = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
    ops.layernorm(normed, x, lw, lb, 1e-5)
    want = [torch.zeros_like(got[0]), torch.zeros_like(got[1]), torch.zeros_like(got[2])]
    ops.gemm_skinny(normed, w, bias, out=want[2], epilogue=ops.EPI_QKV_PAGED, kv=(want[0], want[1], slots, q_dim), ksplit=8, wide=0,
                    mtile=1 if M <= 16 else 0)
    for g, t, what in zip(got, want, ("keys", "values", "queries")):
        if M <= 16:
            assert torch.equal(g, t), what
        else:
            close(g, t, 8e-3, what)
    assert (got[0] == 0).sum() == (want[0] == 0).sum()  # nothing written outside the tokens' slots


@pytest.mark.parametrize("seed", range(4))
def test_drawn_shapes_of_the_folded_and_the_cut_products(ops, seed):
    """Shapes drawn at random (rows, widths that are multiples of 8 only, any number of output
    features, planes up to 16, rows to add to in up to 9 planes): the folded norm against norm +
    product, the cut products against the whole product."""
    import random

    rng = random.Random(seed)
    for _ in range(12):
        M = rng.choice([1, 2, 7, 8, 9, 16, 17, 31, 32])
        K, N, P = 8 * rng.randint(1, 256), rng.randint(1, 700), rng.choice([1, 1, 2, 4, 5, 16])
        planes = rnd(P, M, K, scale=2.0, seed=rng.randint(0, 99))
        planes[0] += 0.5
        x = planes if P > 1 else planes[0]
        lw, lb = rnd(K, seed=5) + 1.0, rnd(K, seed=6)
        w, bias = rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16), rnd(N, seed=2)
        out = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops.gemm_skinny_ln(x, lw, lb, 1e-5, w, bias, out=out, epilogue=ops.EPI_GELU_TANH, wide=rng.choice([0, 1]) if M <= 16 else 0)
        normed = torch.empty(M, K, dtype=torch.bfloat16, device=DEV)
        ops.layernorm(normed, x, lw, lb, 1e-5)
        two = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        ops.gemm(normed, w, bias, out=two, epilogue=ops.EPI_GELU_TANH)
        close(out, two, 1e-2, f"folded norm M={M} K={K} N={N} planes={P}")
    for _ in range(12):
        M, K, N = rng.choice([1, 5, 16, 33, 64]), 8 * rng.randint(8, 400), rng.randint(1, 300)
        units = (K + 63) // 64
        parts = rng.randint(1, min(8, units))
        if (parts - 1) * ((units + parts - 1) // parts) >= units:
            parts = 1
        a, w, bias = rnd(M, K, dtype=torch.bfloat16), rnd(N, K, seed=1, scale=0.2, dtype=torch.bfloat16), rnd(N, seed=2)
        base = rnd(rng.choice([1, 2, 4, 5, 9]), M, N, seed=3)
        want = a.double() @ w.double().t() + bias.double() + base.double().sum(0)
        planes = torch.full((parts, M, N), float("nan"), device=DEV)
        ops.gemm_skinny_parts(a, w, planes, bias=bias, base=base)
        close(planes.double().sum(0), want, 1e-5, f"streaming product in parts M={M} K={K} N={N} parts={parts}")
        if K % 64 == 0 and parts <= K // 64 and (parts - 1) * ((K // 64 + parts - 1) // parts) < K // 64:
            planes = torch.full((parts, M, N), float("nan"), device=DEV)
            ops.gemm_mfma_dl_parts(a, w, planes, bias=bias, base=base, tile=rng.choice([6, 16]))
            close(planes.double().sum(0), want, 1e-5, f"tiled product in parts M={M} K={K} N={N} parts={parts}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,d,indexed", [(1, 16, True), (7, 100, True), (33, 1600, False), (5, 257, True)])
def test_gather_rows(dtype, n, d, indexed):
    """out[r] = x[rows[r]] in the output's dtype; without rows the first n rows."""
    from liyab_amd.kernels import ops

    g = torch.Generator().manual_seed(n * 1000 + d)
    x = torch.randn(n + 9, d, generator=g).to(DEV)
    rows = torch.randint(0, n + 9, (n,), generator=g, dtype=torch.int32).to(DEV) if indexed else None
    out = torch.full((n, d), 7.0, dtype=dtype, device=DEV)
    ops.gather_rows(out, x, rows)
    want = (x[rows.long()] if indexed else x[:n]).to(dtype)
    assert torch.equal(out, want)


@pytest.mark.parametrize("n", [1, 255, 50257 * 3, 4096 * 256 + 5])
def test_scale_in_place(n):
    from liyab_amd.kernels import ops

    x = torch.randn(n, generator=torch.Generator().manual_seed(n)).to(DEV)
    want = x * 0.37
    ops.scale_(x, 0.37)
    assert torch.equal(x, want)
