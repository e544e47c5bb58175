"""The kernels as functions over torch tensors.

Each function checks on the host that shapes, dtypes and layouts are what
its kernel and grid assume, then launches on torch's current stream. Torch
supplies the device memory and the stream; every computation is the
library's own kernel. Nothing here runs without the GPU and the library.
"""

from __future__ import annotations

import ctypes
import struct
from typing import Optional

import torch

from ..errors import KernelError
from . import lib as _lib

F32, BF16 = 0, 1
EPI_NONE, EPI_GELU_TANH, EPI_GELU_ERF, EPI_RESIDUAL = 0, 1, 2, 3
ACTIVATION_EPILOGUE = {"none": EPI_NONE, "gelu_tanh": EPI_GELU_TANH, "gelu_erf": EPI_GELU_ERF}


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return F32
    if dt == torch.bfloat16:
        return BF16
    raise KernelError(f"the kernels take float32 or bfloat16, not {dt}")


_pinned_stream: Optional[int] = None


def _stream() -> int:
    return _pinned_stream if _pinned_stream is not None else torch.cuda.current_stream().cuda_stream


class on_current_stream:
    """Within this context every launch goes to the stream that was current on entry, looked
    up once instead of at every call (a model step makes a couple of hundred launches)."""

    def __enter__(self):
        global _pinned_stream
        self._before = _pinned_stream
        _pinned_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _pinned_stream
        _pinned_stream = self._before
        return False


_invariant = False


class batch_invariant:
    """Within this context the kernels that serve a row are chosen from the model's sizes and the
    row's own position only, never from what else the step holds: products by the tiled
    matrix-core kernels whose sums run over k in one order whatever the tile (no streaming kernel,
    no cut over K, no norm folded into a product), attention token by token with one split on
    four waves. A row's bfloat16 results then have the same bits alone and in any batch, as the
    reference promises of its passes (include/liyab/engine.h:987-990, src/core/transformer.h:746-751);
    the step-shaped choices outside this context are faster and differ from these by rounding."""

    def __init__(self, on: bool = True):
        self.on = on

    def __enter__(self):
        global _invariant
        self._before = _invariant
        _invariant = self.on
        return self

    def __exit__(self, *exc):
        global _invariant
        _invariant = self._before
        return False


def is_batch_invariant() -> bool:
    return _invariant


def _dev(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise KernelError(f"{what} must be on the GPU")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _i32(t: torch.Tensor, what: str, n: Optional[int] = None, pinned_ok: bool = False) -> None:
    if not (pinned_ok and not t.is_cuda and t.is_pinned()):  # (pinned host memory is mapped into the device's address space)
        _dev(t, what)
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what} must be contiguous int32")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what} holds {t.numel()} values, {n} are needed")


def _f32vec(t: Optional[torch.Tensor], what: str, n: int) -> None:
    if t is None:
        return
    _dev(t, what)
    if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != n:
        raise KernelError(f"{what} must be {n} contiguous float32 values, got {tuple(t.shape)} {t.dtype}")


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    _dev(t, what)
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{what} must be 2-D with contiguous rows, got shape {tuple(t.shape)} strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _pages(k_cache: torch.Tensor, num_pages: Optional[int]) -> int:
    """The number of pages a launcher is told the caches hold: all of them unless the caller
    counts fewer (page ids and slots beyond that count are not followed by the kernels)."""
    pages = k_cache.shape[0] if num_pages is None else int(num_pages)
    if not 0 < pages <= k_cache.shape[0]:
        raise KernelError(f"the caches hold {k_cache.shape[0]} pages, not {pages}")
    if pages * k_cache.shape[2] >= 1 << 31:
        raise KernelError(f"{pages} pages of {k_cache.shape[2]} positions: slots must fit 31 bits")
    return pages


def check_device() -> None:
    _lib.call("liyab_check_device")


def fill_(t: torch.Tensor, value: float | int) -> torch.Tensor:
    _dev(t, "fill target")
    if not t.is_contiguous():
        raise KernelError("fill target must be contiguous")
    if t.dtype == torch.float32:
        bits = struct.unpack("<I", struct.pack("<f", float(value)))[0]
        size = 4
    elif t.dtype == torch.int32:
        bits = int(value) & 0xFFFFFFFF
        size = 4
    elif t.dtype == torch.bfloat16:
        bits = struct.unpack("<I", struct.pack("<f", float(value)))[0]
        bits = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) & 0xFFFF if value == value else 0x7FC0
        size = 2
    else:
        raise KernelError(f"fill: unsupported dtype {t.dtype}")
    _lib.call("liyab_fill", t.data_ptr(), size, bits, t.numel(), _stream())
    return t


def add_into_(residual: torch.Tensor, x: torch.Tensor) -> None:
    """residual (float32) += x, elementwise."""
    _dev(residual, "residual")
    _dev(x, "x")
    if residual.dtype != torch.float32 or not residual.is_contiguous() or not x.is_contiguous():
        raise KernelError("add_into: residual must be contiguous float32 and x contiguous")
    if residual.numel() != x.numel():
        raise KernelError(f"add_into: {residual.numel()} vs {x.numel()} values")
    _lib.call("liyab_add_into", residual.data_ptr(), x.data_ptr(), dtype_code(x.dtype), x.numel(), _stream())


def embed(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0,
          pos_table: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None,
          last_tokens: Optional[torch.Tensor] = None) -> None:
    """out[t] = scale * table[ids[t]] (+ pos_table[positions[t]]); out is float32 [n, d].
    An id below zero stands for last_tokens[-1 - id]. The caller has checked ids against the
    table's rows (and positions against pos_table's)."""
    _dev(out, "out")
    n, d = out.shape
    if out.dtype != torch.float32 or not out.is_contiguous():
        raise KernelError("embed: out must be contiguous float32")
    if table.dim() != 2 or table.shape[1] != d or not table.is_contiguous():
        raise KernelError(f"embed: table {tuple(table.shape)} does not have rows of {d}")
    _i32(ids, "ids", n)
    if pos_table is not None:
        if pos_table.dtype != table.dtype or pos_table.dim() != 2 or pos_table.shape[1] != d or not pos_table.is_contiguous():
            raise KernelError("embed: the position table must match the token table's dtype and width")
        if positions is None:
            raise KernelError("embed: a position table needs positions")
        _i32(positions, "positions", n)
    if last_tokens is not None:
        _i32(last_tokens, "last_tokens")
    _lib.call("liyab_embed", out.data_ptr(), table.data_ptr(), _ptr(pos_table), dtype_code(table.dtype),
              ids.data_ptr(), _ptr(positions), n, d, float(scale), _ptr(last_tokens), _stream())


def add_rows_(x: torch.Tensor, table: torch.Tensor, rows: torch.Tensor) -> None:
    """x[t] += table[rows[t]]; x is float32 [n, d]."""
    _dev(x, "x")
    n, d = x.shape
    if x.dtype != torch.float32 or not x.is_contiguous():
        raise KernelError("add_rows: x must be contiguous float32")
    if table.dim() != 2 or table.shape[1] != d or not table.is_contiguous():
        raise KernelError(f"add_rows: table {tuple(table.shape)} does not have rows of {d}")
    _i32(rows, "rows", n)
    _lib.call("liyab_add_rows", x.data_ptr(), table.data_ptr(), dtype_code(table.dtype), rows.data_ptr(), n, d, _stream())


def gather_rows(out: torch.Tensor, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = x[rows[r]] (x[r] without rows) in out's dtype; x float32 [*, d], out [n, d]."""
    _dev(out, "out")
    _dev(x, "x")
    n, d = out.shape
    if x.dtype != torch.float32 or x.dim() != 2 or x.shape[1] != d or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"gather_rows: x must be contiguous float32 [*, {d}] and out contiguous, got {tuple(x.shape)} {x.dtype}")
    if rows is not None:
        _i32(rows, "rows", n)
    elif x.shape[0] < n:
        raise KernelError("gather_rows: fewer input rows than output rows")
    _lib.call("liyab_gather_rows", out.data_ptr(), dtype_code(out.dtype), x.data_ptr(), _ptr(rows), n, d, _stream())


def scale_(t: torch.Tensor, scale: float) -> torch.Tensor:
    """t *= scale; t contiguous float32."""
    _dev(t, "scale target")
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise KernelError("scale: the target must be contiguous float32")
    _lib.call("liyab_scale", t.data_ptr(), float(scale), t.numel(), _stream())
    return t


def _planes(x: torch.Tensor, what: str):
    """Rows given as they are, float32 [rows, d], or as a sum of planes, float32 [parts, rows, d]
    (row r is x[0][r] + x[1][r] + ..., added in that order). Returns (pointer, parts, floats
    between planes, rows, d)."""
    _dev(x, what)
    if x.dtype != torch.float32 or x.dim() not in (2, 3) or not x.is_contiguous():
        raise KernelError(f"{what}: rows must be contiguous float32 [rows, d] or [parts, rows, d], got {tuple(x.shape)} {x.dtype}")
    if x.dim() == 2:
        return x.data_ptr(), 1, 0, x.shape[0], x.shape[1]
    if not 1 <= x.shape[0] <= 16:
        raise KernelError(f"{what}: {x.shape[0]} planes (1 to 16)")
    return x.data_ptr(), x.shape[0], x.stride(0), x.shape[1], x.shape[2]


def norm_takes_planes(d: int) -> bool:
    """Whether the norm kernel adds planes up as it loads a row of this width (sum_parts first otherwise)."""
    return d % 4 == 0 and d <= 16384


def layernorm(out: torch.Tensor, x: torch.Tensor, weight: Optional[torch.Tensor], bias: Optional[torch.Tensor],
              eps: float, rows: Optional[torch.Tensor] = None) -> None:
    """out[r] = LayerNorm(x[rows[r]] or x[r]); x float32 [*, d], out [n, d] float32 or bfloat16.
    x may be a sum of planes [parts, *, d] (widths that `norm_takes_planes`): the planes are
    added up, in their order, as a row is loaded."""
    _dev(out, "out")
    ptr, n_parts, stride, x_rows, xd = _planes(x, "layernorm")
    n, d = out.shape
    if xd != d or not out.is_contiguous():
        raise KernelError("layernorm: x must have rows of d and out must be contiguous [n, d]")
    _f32vec(weight, "norm weight", d)
    _f32vec(bias, "norm bias", d)
    if rows is not None:
        _i32(rows, "rows", n)
    elif x_rows < n:
        raise KernelError("layernorm: fewer input rows than output rows")
    if n_parts == 1:
        _lib.call("liyab_layernorm", out.data_ptr(), dtype_code(out.dtype), ptr, _ptr(weight), _ptr(bias),
                  _ptr(rows), n, d, float(eps), _stream())
        return
    _lib.call("liyab_layernorm_parts", out.data_ptr(), dtype_code(out.dtype), ptr, n_parts, stride, x_rows, _ptr(weight),
              _ptr(bias), _ptr(rows), n, d, float(eps), _stream())


def sum_parts(out: torch.Tensor, planes: torch.Tensor) -> None:
    """out = planes[0] + planes[1] + ..., in the order the norm kernels add them; out float32
    [rows, d] (it may be planes[0])."""
    _dev(out, "out")
    ptr, n_parts, stride, x_rows, d = _planes(planes, "sum_parts")
    if out.dtype != torch.float32 or tuple(out.shape) != (x_rows, d) or not out.is_contiguous():
        raise KernelError(f"sum_parts: out must be contiguous float32 [{x_rows}, {d}]")
    _lib.call("liyab_sum_parts", out.data_ptr(), x_rows, d, ptr, n_parts, stride, _stream())


def gemm_simple(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out: Optional[torch.Tensor] = None,
                residual: Optional[torch.Tensor] = None, epilogue: int = EPI_NONE) -> None:
    """out = epilogue(a . w^T + bias), or residual += a . w^T + bias.
    a [M, K] and w [N, K] share a dtype; rows of a and out may be strided."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    if w.dim() != 2 or w.shape[1] != K or not w.is_contiguous() or w.dtype != a.dtype:
        raise KernelError(f"gemm: w {tuple(w.shape)} {w.dtype} does not fit a {tuple(a.shape)} {a.dtype}")
    N = w.shape[0]
    _f32vec(bias, "bias", N)
    ldo = ldr = 0
    out_code = F32
    if epilogue == EPI_RESIDUAL:
        if residual is None or residual.dtype != torch.float32 or tuple(residual.shape) != (M, N):
            raise KernelError("gemm: the residual epilogue needs a float32 residual [M, N]")
        ldr = _rows(residual, "residual")
    else:
        if out is None or tuple(out.shape) != (M, N):
            raise KernelError("gemm: out must be [M, N]")
        ldo = _rows(out, "out")
        out_code = dtype_code(out.dtype)
    _lib.call("liyab_gemm_simple", _ptr(out), out_code, ldo, a.data_ptr(), lda, w.data_ptr(), dtype_code(a.dtype),
              _ptr(bias), _ptr(residual), ldr, M, N, K, epilogue, _stream())


def kv_write(k_cache: torch.Tensor, v_cache: torch.Tensor, src: torch.Tensor, k_off: int, v_off: int,
             slots: torch.Tensor, num_pages: Optional[int] = None) -> None:
    """Writes token t's keys src[t, k_off:k_off+Hkv*hd] and values to slot slots[t] of caches
    laid out [pages, kv_heads, page_size, head_dim]. Slots are page * page_size + offset; a
    slot outside the caches' `num_pages` (all of them by default) pages is not written."""
    _dev(k_cache, "k_cache")
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("kv_write: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
    if src.dtype != k_cache.dtype or v_cache.dtype != k_cache.dtype:
        raise KernelError("kv_write: source and caches must share a dtype")
    stride = _rows(src, "src")
    n = src.shape[0]
    _i32(slots, "slots", n)
    _, hkv, page, hd = k_cache.shape
    if k_off + hkv * hd > src.shape[1] or v_off + hkv * hd > src.shape[1]:
        raise KernelError("kv_write: column offsets pass the source's width")
    _lib.call("liyab_kv_write", k_cache.data_ptr(), v_cache.data_ptr(), src.data_ptr(), dtype_code(src.dtype), stride,
              k_off, v_off, slots.data_ptr(), n, hkv, hd, page, _pages(k_cache, num_pages), _stream())


def attention_generic(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor, *, n_head: int,
                      scale: float, window: int = 0, num_pages: Optional[int] = None) -> None:
    """out[t, h*hd:(h+1)*hd] = softmax(scale * q_th . K[:pos_t+1]) V for the request tok_seq[t].
    q is [n, >= n_head*hd] (a view into a wider projection output is fine)."""
    n = out.shape[0]
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
    _, hkv, page, hd = k_cache.shape
    os_ = _rows(out, "out")
    qs = _rows(q, "q")
    if q.shape[0] != n or q.shape[1] < n_head * hd or out.shape[1] != n_head * hd:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {n_head} heads of {hd}")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
        raise KernelError("attention: q, out and the caches must share a dtype")
    _dev(block_tables, "block_tables")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise KernelError("attention: block_tables must be contiguous int32 [requests, max_blocks]")
    _i32(tok_seq, "tok_seq", n)
    _i32(tok_pos, "tok_pos", n)
    _lib.call("liyab_attention_generic", out.data_ptr(), os_, q.data_ptr(), qs, k_cache.data_ptr(), v_cache.data_ptr(),
              dtype_code(q.dtype), block_tables.data_ptr(), block_tables.shape[1], tok_seq.data_ptr(),
              tok_pos.data_ptr(), n, float(scale), int(window), n_head, hkv, hd, page, _pages(k_cache, num_pages), _stream())


_argmax_scratch = {}


def _scatter(scatter, rows):
    if scatter is None:
        return None, None
    index, target = scatter
    _i32(index, "scatter index", rows)
    _i32(target, "scatter target")
    return index.data_ptr(), target.data_ptr()


def argmax(out: torch.Tensor, logits: torch.Tensor, scatter=None) -> None:
    """out[r] = the first maximal element of logits[r] (ties go to the lowest id). With
    scatter = (index, target), target[index[r]] = out[r] too; the caller has checked the
    indices against the target. `out` may be pinned host memory: the kernel then writes the
    tokens where the host reads them, and no copy follows."""
    ld = _rows(logits, "logits")
    rows, V = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("argmax: logits must be float32")
    _i32(out, "out", rows, pinned_ok=True)
    key = logits.device
    sc = _argmax_scratch.get(key)
    if sc is None or sc[0].numel() < rows * 64:
        cap = max(rows, 64) * 64
        sc = (torch.empty(cap, dtype=torch.float32, device=key), torch.empty(cap, dtype=torch.int32, device=key))
        _argmax_scratch[key] = sc
    si, so = _scatter(scatter, rows)
    _lib.call("liyab_argmax", out.data_ptr(), logits.data_ptr(), ld, rows, V, sc[0].data_ptr(), sc[1].data_ptr(), si, so,
              _stream())


def sample(out: torch.Tensor, logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor,
           top_p: torch.Tensor, uniform: torch.Tensor, scatter=None) -> None:
    """Per-row sampling; temperature/top_p float32 [rows], top_k int32 [rows], uniform float64 [rows] in [0, 1).
    top_k and top_p may both be None when no row cuts its candidates: a shorter kernel runs then.
    `out` may be pinned host memory, as for `argmax`."""
    ld = _rows(logits, "logits")
    rows, V = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("sample: logits must be float32")
    _i32(out, "out", rows, pinned_ok=True)
    _f32vec(temperature, "temperature", rows)
    if (top_k is None) != (top_p is None):
        raise KernelError("sample: top_k and top_p are given together or not at all")
    if top_k is not None:
        _f32vec(top_p, "top_p", rows)
        _i32(top_k, "top_k", rows)
    _dev(uniform, "uniform")
    if uniform.dtype != torch.float64 or uniform.numel() != rows or not uniform.is_contiguous():
        raise KernelError("sample: uniform must be contiguous float64 [rows]")
    si, so = _scatter(scatter, rows)
    _lib.call("liyab_sample", out.data_ptr(), logits.data_ptr(), ld, rows, V, temperature.data_ptr(),
              0 if top_k is None else top_k.data_ptr(), 0 if top_p is None else top_p.data_ptr(),
              uniform.data_ptr(), si, so, _stream())


EPI_QKV_PAGED = 4


class _Rows:
    """What `_epilogue` reads of a first operand that is no tensor: its rows and its dtype."""

    def __init__(self, rows: int, dtype: torch.dtype):
        self.shape, self.dtype = (rows, 0), dtype


def _epilogue(a, w, bias, out, residual, epilogue, kv):
    """Checks the epilogue's operands against [M, N] and fills the launchers' struct."""
    M, N = a.shape[0], w.shape[0]
    _f32vec(bias, "bias", N)
    e = _lib.EpiParams()
    e.mode = epilogue
    e.bias = _ptr(bias)
    e.exact = 1 if a.dtype == torch.float32 else 0
    e.out_dtype = F32
    if epilogue == EPI_RESIDUAL:
        if residual is None or residual.dtype != torch.float32 or tuple(residual.shape) != (M, N):
            raise KernelError("gemm: the residual epilogue needs a float32 residual [M, N]")
        e.residual, e.ldr = residual.data_ptr(), _rows(residual, "residual")
    elif epilogue == EPI_QKV_PAGED:
        k_cache, v_cache, slots, q_dim = kv[:4]
        e.num_slots = _pages(k_cache, kv[4] if len(kv) > 4 else None) * k_cache.shape[2]
        if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
            raise KernelError("gemm: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
        _, hkv, page, hd = k_cache.shape
        if out is None or tuple(out.shape) != (M, q_dim) or q_dim + 2 * hkv * hd != N:
            raise KernelError(f"gemm: the paged QKV epilogue needs out [M, {q_dim}] and N = q_dim + 2 * kv_dim")
        if not (out.dtype == k_cache.dtype == v_cache.dtype):
            raise KernelError("gemm: queries and caches must share a dtype")
        _i32(slots, "slots", M)
        e.out, e.ldo, e.out_dtype = out.data_ptr(), _rows(out, "out"), dtype_code(out.dtype)
        e.kc, e.vc, e.slots = k_cache.data_ptr(), v_cache.data_ptr(), slots.data_ptr()
        e.q_dim, e.kv_dim, e.hd, e.n_kv_head, e.page_size = q_dim, hkv * hd, hd, hkv, page
    else:
        if out is None or tuple(out.shape) != (M, N):
            raise KernelError("gemm: out must be [M, N]")
        e.out, e.ldo, e.out_dtype = out.data_ptr(), _rows(out, "out"), dtype_code(out.dtype)
    return e


def gemm_mfma(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out=None, residual=None,
              epilogue: int = EPI_NONE, kv=None, tile: int = 0) -> None:
    """The matrix-core product for bfloat16 operands with K a multiple of 8."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_mfma: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    e = _epilogue(a, w, bias, out, residual, epilogue, kv)
    _lib.call("liyab_gemm_mfma", a.data_ptr(), lda, w.data_ptr(), M, w.shape[0], K, tile, ctypes.byref(e), _stream())


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out=None, residual=None,
                epilogue: int = EPI_NONE, kv=None, ksplit: int = 0, wide: int = -1, mtile: int = 0) -> None:
    """The weight-streaming product for at most 64 bfloat16 rows, K a multiple of 8. ksplit
    (waves sharing K), wide (64 output features a workgroup) and mtile (tiles of 16 rows a
    workgroup) are chosen from the shape unless given."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_skinny: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    if M > 64:
        raise KernelError(f"gemm_skinny: {M} rows; it takes at most 64")
    e = _epilogue(a, w, bias, out, residual, epilogue, kv)
    _lib.call("liyab_gemm_skinny", a.data_ptr(), lda, w.data_ptr(), M, w.shape[0], K, ksplit, wide, mtile, ctypes.byref(e), _stream())


def gemm_skinny_parts(a: torch.Tensor, w: torch.Tensor, planes: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
                      base: Optional[torch.Tensor] = None, ksplit: int = 0) -> None:
    """planes[p] = a . w^T summed over the p-th of planes.shape[0] parts of K: the
    weight-streaming product cut over K, for few output features and a long K. a [M <= 64, K]
    and w [N, K] bfloat16, planes float32 [parts, M, N]. With `base` (float32 [M, N] or a sum
    of planes [*, M, N], not overlapping `planes`) the first plane also takes `bias` and the
    rows of `base`, so that the planes add up to base + a . w^T + bias."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    _dev(planes, "planes")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_skinny_parts: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    N = w.shape[0]
    if planes.dtype != torch.float32 or planes.dim() != 3 or tuple(planes.shape[1:]) != (M, N) or not planes.is_contiguous():
        raise KernelError(f"gemm_skinny_parts: planes must be contiguous float32 [parts, {M}, {N}], got {tuple(planes.shape)}")
    bptr, n_base, bstride = None, 0, 0
    if base is not None:
        bptr, n_base, bstride, b_rows, b_d = _planes(base, "gemm_skinny_parts: base")
        if (b_rows, b_d) != (M, N):
            raise KernelError(f"gemm_skinny_parts: base must have rows [{M}, {N}], got {tuple(base.shape)}")
        _f32vec(bias, "bias", N)
    elif bias is not None:
        raise KernelError("gemm_skinny_parts: a bias needs the rows it is added to (base)")
    _lib.call("liyab_gemm_skinny_parts", a.data_ptr(), lda, w.data_ptr(), M, N, K, planes.shape[0], ksplit,
              planes.data_ptr(), planes.stride(0), _ptr(bias), bptr, n_base, bstride, _stream())


def gemm_mfma_dl_parts(a: torch.Tensor, w: torch.Tensor, planes: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
                       base: Optional[torch.Tensor] = None, tile: int = 6) -> None:
    """The tiled matrix-core product cut over K (K a multiple of 64), as `gemm_skinny_parts` for
    any number of rows: planes float32 [parts, M, N]; with `base` the first plane also takes
    `bias` and the rows of `base`. tile: 6 = 64 x 64 tiles, 16 = 64 x 32, 17 = 32 x 32."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    _dev(planes, "planes")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_mfma_dl_parts: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    N = w.shape[0]
    if planes.dtype != torch.float32 or planes.dim() != 3 or tuple(planes.shape[1:]) != (M, N) or not planes.is_contiguous():
        raise KernelError(f"gemm_mfma_dl_parts: planes must be contiguous float32 [parts, {M}, {N}], got {tuple(planes.shape)}")
    bptr, n_base, bstride = None, 0, 0
    if base is not None:
        bptr, n_base, bstride, b_rows, b_d = _planes(base, "gemm_mfma_dl_parts: base")
        if (b_rows, b_d) != (M, N):
            raise KernelError(f"gemm_mfma_dl_parts: base must have rows [{M}, {N}], got {tuple(base.shape)}")
        _f32vec(bias, "bias", N)
    elif bias is not None:
        raise KernelError("gemm_mfma_dl_parts: a bias needs the rows it is added to (base)")
    _lib.call("liyab_gemm_mfma_dl_parts", a.data_ptr(), lda, w.data_ptr(), M, N, K, planes.shape[0], tile,
              planes.data_ptr(), planes.stride(0), _ptr(bias), bptr, n_base, bstride, _stream())


def gemm_att_parts(partials: torch.Tensor, w: torch.Tensor, planes: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
                   base: Optional[torch.Tensor] = None) -> None:
    """The product cut over K (as `gemm_skinny_parts`) whose first operand is attention's output
    still in splits: partials float32 [M <= 32, heads, splits <= 8, head size + 4] as
    `attention_decode(..., leave_splits=True)` leaves them, merged as they are loaded.
    w [N, heads * head size] bfloat16, planes float32 [parts, M, N]."""
    _dev(partials, "partials")
    _dev(w, "w")
    _dev(planes, "planes")
    if partials.dtype != torch.float32 or partials.dim() != 4 or not partials.is_contiguous():
        raise KernelError(f"gemm_att_parts: partials must be contiguous float32 [M, heads, splits, head size + 4], got {tuple(partials.shape)}")
    M, H, S, hd4 = partials.shape
    K = H * (hd4 - 4)
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_att_parts: needs contiguous bfloat16 w [N, {K}], got {tuple(w.shape)} {w.dtype}")
    N = w.shape[0]
    if not att_parts_takes(M, S, hd4 - 4):
        raise KernelError(f"gemm_att_parts: {M} rows in {S} splits of heads of {hd4 - 4} are outside what it takes")
    if planes.dtype != torch.float32 or planes.dim() != 3 or tuple(planes.shape[1:]) != (M, N) or not planes.is_contiguous():
        raise KernelError(f"gemm_att_parts: planes must be contiguous float32 [parts, {M}, {N}], got {tuple(planes.shape)}")
    bptr, n_base, bstride = None, 0, 0
    if base is not None:
        bptr, n_base, bstride, b_rows, b_d = _planes(base, "gemm_att_parts: base")
        if (b_rows, b_d) != (M, N):
            raise KernelError(f"gemm_att_parts: base must have rows [{M}, {N}], got {tuple(base.shape)}")
        _f32vec(bias, "bias", N)
    elif bias is not None:
        raise KernelError("gemm_att_parts: a bias needs the rows it is added to (base)")
    _lib.call("liyab_gemm_att_parts", partials.data_ptr(), S, H, hd4 - 4, w.data_ptr(), M, N, planes.shape[0],
              planes.data_ptr(), planes.stride(0), _ptr(bias), bptr, n_base, bstride, _stream())


def att_parts_takes(M: int, splits: int, hd: int) -> bool:
    return 0 < M <= 32 and 1 <= splits <= 8 and hd % 8 == 0 and 8 <= hd <= 256


def k_parts(M: int, N: int, K: int) -> int:
    """Into how many parts of K the weight-streaming product is best cut (1: not at all). With
    few output features a product fills a fraction of the chip's compute units, and a long K
    then streams through those few; cut over K it covers the chip. Measured at 8 rows, whole
    and in parts (us): 3,072 -> 768 7.2 and 4.5 (four parts), 768 -> 768 4.6 and 3.4 (four),
    6,400 -> 1,600 13.4 and 8.5 (two), 1,600 -> 1,600 5.4 and 4.6 (two)."""
    if M > 32 or K % 8 != 0 or _invariant:
        return 1
    groups, units = (N + 15) // 16 * ((M + 15) // 16), (K + 63) // 64  # workgroups uncut; units of 64 k
    parts = 1
    while parts < 4 and groups * parts * 2 <= 256 and units // (parts * 2) >= 3:
        parts *= 2
    return parts


def skinny_parts_takes(M: int, N: int, K: int) -> bool:
    """Whether `gemm_skinny_parts` takes this shape and is the kernel `gemm` would choose for it."""
    return 0 < M <= 64 and K % 8 == 0 and N <= 8192 and not (M > 32 and K % 64 == 0 and N >= 2048)


def tiled_k_parts(M: int, N: int, K: int) -> int:
    """Into how many parts of K the tiled product of more than 32 rows (of more than 16, with many
    output features) is best cut when it is added to the residual stream (1: not at all).
    Several tiles of rows, few output features and a long K (a prompt's portion through the feed-forward's second product: 128 x 768 x 3,072 is
    24 tiles of 64 x 64, each walking the whole of K in 18.7 us): cut until the tiles cover the
    chip. One tile of rows (33 to 64): the 64 x 32 tiles are few and each walks the whole of K;
    cut over K they cover the chip: alone, at 64 rows, 3,072 -> 768 takes 8.2 us whole (the streaming kernel) and 4.9 in 8 parts, 6,400 ->
    1,600 19.8 and 8.2. In a decode step the next readers pay for the planes, though: inner
    dimensions from 3,072 gain, in 4 parts (ms a step at 64 rows, whole and cut: GPT-2 small's
    sizes 0.806 and 0.797, medium's 1.767 and 1.715; XL's 5.19 and 4.90)."""
    if K % 64 != 0 or M <= 16 or _invariant:
        return 1
    if M <= 64:
        if N <= 2048:
            return 4 if K >= 3072 and M > 32 else 1
        # more output features: the largest tiles that take the rows in one, 32 x 32 up to 32 rows and
        # 64 x 64 beyond (every tile reads all the rows: at 64 rows, 32 x 32 tiles read them twice as
        # often as the weights), cut while tiles x parts stay within the chip (us alone, whole as it
        # was and cut: 64 rows, 16,384 -> 4,096 42.2 and 32.3 in 4 parts, 4,096 -> 4,096 13.5 and 9.7,
        # 8,192 -> 8,192 34.8 and 31.6 in 2 parts; 32 rows, 16,384 -> 4,096 39.7 and 27.8 in 2 parts,
        # 4,096 -> 4,096 12.3 and 9.6, 8,192 -> 8,192 27.3 whole)
        side = 32 if M <= 32 else 64
        tiles, parts = (N + side - 1) // side, 1
        while parts < 4 and tiles * parts * 2 <= 256 and K // 64 // (parts * 2) >= 8:  # (256: the compute units of the part this was measured on)
            parts *= 2
        return parts
    # several tiles of rows (a prompt's portion): 64 x 64 tiles, cut until they cover the chip,
    # a part keeping 256 of K or more; in two parts while two workgroups a compute unit hold them
    # (ms a step of 768 / 1,024 tokens whole and in two parts: GPT-2 small's sizes 1.00 and 0.99 /
    # 1.13 and 1.12, medium's 2.32 and 2.16 / 2.54 and 2.47; XL's at 512 tokens 6.11 and 5.88)
    tiles = (M + 63) // 64 * ((N + 63) // 64)
    nk = K // 64
    parts = 1
    while parts < TILED_MAX_PARTS and tiles * parts * 2 <= (512 if parts == 1 else 256) and nk // (parts * 2) >= 4:
        parts *= 2
    return parts


TILED_MAX_PARTS = 4  # (us a step of 128 / 256 / 512 tokens of one prompt with at most 1, 2, 4, 8 parts: 765 665 637 668 / 809 720 694 679 / 922 843 842 846)


def gemm_skinny_ln(x: torch.Tensor, ln_weight: Optional[torch.Tensor], ln_bias: Optional[torch.Tensor], eps: float,
                   w: torch.Tensor, bias: Optional[torch.Tensor], *, out=None, epilogue: int = EPI_NONE, kv=None,
                   wide: int = -1) -> None:
    """The weight-streaming product over LayerNorm(x) of the float32 rows x [M, K], or of a sum
    of planes [parts, M, K], the norm computed inside the product kernel (`skinny_ln_takes`).
    wide: 32 instead of 16 output features a workgroup (-1: chosen from the shape)."""
    ptr, n_parts, stride, M, K = _planes(x, "gemm_skinny_ln")
    _dev(w, "w")
    if w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_skinny_ln: needs contiguous bfloat16 w [N, {K}], got {tuple(w.shape)} {w.dtype}")
    if not skinny_ln_takes(M, K):
        raise KernelError(f"gemm_skinny_ln: {M} rows of {K} are outside what it takes")
    if epilogue == EPI_RESIDUAL:
        raise KernelError("gemm_skinny_ln: the residual epilogue is not taken")
    _f32vec(ln_weight, "norm weight", K)
    _f32vec(ln_bias, "norm bias", K)
    e = _epilogue(_Rows(M, torch.bfloat16), w, bias, out, None, epilogue, kv)
    e.exact = 0
    _lib.call("liyab_gemm_skinny_ln", ptr, n_parts, stride, _ptr(ln_weight), _ptr(ln_bias), float(eps),
              w.data_ptr(), M, w.shape[0], K, wide, ctypes.byref(e), _stream())


def skinny_ln_takes(M: int, K: int) -> bool:
    """What the product kernel with the norm inside takes: one or two tiles of 16 rows, a row in
    a wave's registers."""
    return 0 < M <= 32 and K % 8 == 0 and K <= 2048


_compute_units = 0


def compute_units() -> int:
    global _compute_units
    if not _compute_units:
        _compute_units = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    return _compute_units


def skinny_ln_pays(M: int, N: int, K: int) -> bool:
    """Whether folding the norm into the product beats the norm kernel followed by the plain
    product. The folded kernel keeps a row in registers, so one workgroup fills a compute unit:
    with more workgroups (16 or 32 output features each) than compute units they run in two
    rounds, which costs more than the norm's kernel (GPT-2 XL's 1,600 -> 4,800 at 8 rows in
    strips of 16: 15.2 us folded against 9 + 4.5)."""
    return not _invariant and skinny_ln_takes(M, K) and (N + (31 if M <= 16 else 15)) // (32 if M <= 16 else 16) <= compute_units()


def gemm_mfma_dl(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out=None, residual=None,
                 epilogue: int = EPI_NONE, kv=None, tile: int = 0) -> None:
    """The matrix-core product with tiles loaded straight into LDS, three stages deep; bfloat16
    operands, K a multiple of 64."""
    lda = _rows(a, "a")
    M, K = a.shape
    _dev(w, "w")
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or w.dim() != 2 or w.shape[1] != K or not w.is_contiguous():
        raise KernelError(f"gemm_mfma_dl: needs bfloat16 a [M, K] and contiguous w [N, K], got {tuple(a.shape)} {a.dtype}, {tuple(w.shape)} {w.dtype}")
    if K % 64 != 0 or M == 0:
        raise KernelError(f"gemm_mfma_dl: K = {K} must be a multiple of 64 and M positive")
    e = _epilogue(a, w, bias, out, residual, epilogue, kv)
    _lib.call("liyab_gemm_mfma_dl", a.data_ptr(), lda, w.data_ptr(), M, w.shape[0], K, tile, ctypes.byref(e), _stream())


def mfma_takes(a: torch.Tensor, w: torch.Tensor) -> bool:
    return (a.dtype == torch.bfloat16 and a.shape[1] % 8 == 0 and a.stride(0) % 8 == 0 and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def gemm(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out: Optional[torch.Tensor] = None,
         residual: Optional[torch.Tensor] = None, epilogue: int = EPI_NONE, kv=None) -> None:
    """The product kernel for these operands: matrix cores for bfloat16 shapes they take,
    the plain tiled kernel for float32 and everything else. `kv` = (k_cache, v_cache, slots,
    q_dim[, num_pages]) with the paged QKV epilogue (a slot outside the caches' pages is not written)."""
    if _invariant and mfma_takes(a, w):
        # one family of kernels whatever the number of rows: their sum over k has one order for
        # every tile shape, so a row's bits do not depend on the rows beside it. K a multiple of 64:
        # four sums, unit u of 64 k going to sum u % 4 (16 k an instruction), added in their order;
        # up to 64 rows four groups of waves walk K side by side, a sum each, in small tiles that
        # cover the chip; more rows take the large tiles, whose one group keeps the four sums.
        M, N, K = a.shape[0], w.shape[0], a.shape[1]
        if K % 64 == 0:
            if M <= 64:
                tile = 17 if M <= 32 or 2 * ((N + 31) // 32) <= compute_units() else 16
            else:
                tile = 108 if M * N >= 2048 * 2048 else (106 if K >= 2048 else 102)
            gemm_mfma_dl(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, tile=tile)
        else:
            gemm_mfma(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, tile=2)
        return
    if mfma_takes(a, w):
        M, N = a.shape[0], w.shape[0]
        if 12 < M <= 128 and N >= 16384 and a.shape[1] % 64 == 0 and (N + 127) // 128 >= compute_units():
            # a vocabulary's worth of output features: large tiles re-read the tokens least
            # (16 rows: 22.5 against 25.1 us for 768 -> 50,257; 64 rows: 27.9 against 32.9); with fewer such tiles
            # than compute units they stream too slowly (4,096 -> 16,384 at 64 rows: 128 tiles, 65 us)
            gemm_mfma_dl(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, tile=8)
        elif ((M > 32 or (M > 16 and N * a.shape[1] >= 6 << 20)) and a.shape[1] % 64 == 0 and N >= 2048
              and (M + 63) // 64 * ((N + 31) // 32) <= compute_units()):
            # one tile of 33 to 64 rows and many output features: 64 x 32 tiles share the tokens'
            # rows through LDS where the streaming kernel's workgroups each read them again (40
            # rows: 5.2 against 6.4 us for 768 -> 2,304, 8.0 against 10.4 for 1,600 -> 4,800; the
            # products back to the model's width, with fewer tiles, stay with the streaming kernel);
            # the largest matrices already from 17 rows (32 rows, weights cold from HBM: 8.9
            # against 12.5 us for 1,600 -> 4,800, but 6.6 against 6.1 for 1,024 -> 3,072); more
            # tiles of rows as long as every tile has a compute unit of its own (the stages fill
            # a unit's LDS; 128 rows: 6.1 against 7.7 us for 768 -> 2,304 in 64 x 64 tiles; with
            # more tiles than units, 400 rows: 10.7 against 8.0)
            # tiles of 32 x 32 while each has a compute unit of its own: a workgroup brings in a third
            # less of the operands and twice as many pull (64 rows, cold weights: 5.05 against 5.53 us
            # for 768 -> 2,304, 5.97 against 6.85 for 1,024 -> 3,072; 13.9 against 9.7 for 1,600 -> 4,800)
            small = (M + 31) // 32 * ((N + 31) // 32) <= compute_units()
            gemm_mfma_dl(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, tile=17 if small else 16)
        elif M <= 16 or (M <= 64 and N <= 8192):
            # few tokens: stream the weights (for a huge N and more than 16 tokens the tiled
            # kernel's shared loads beat every workgroup re-reading the tokens); 11 to 16 tokens and
            # very many output features in strips of 64, which read the tokens a quarter as often (16
            # rows, alone: 4,096 -> 16,384 31.6 against 36.4 us, -> 12,288 25.3 against 28.5; at 8 rows
            # and at 6,400 features strips of 16 win)
            gemm_skinny(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv, wide=1 if 10 < M <= 16 and N >= 12288 else 0)
        elif a.shape[1] % 64 == 0:
            gemm_mfma_dl(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv)
        else:
            gemm_mfma(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv)
        return
    if epilogue == EPI_QKV_PAGED:
        # the plain kernel writes the whole projection; a second kernel moves keys and values
        raise KernelError("gemm: the paged QKV epilogue is for the matrix-core kernels; use gemm + kv_write")
    gemm_simple(a, w, bias, out=out, residual=residual, epilogue=epilogue)


def attention_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     block_tables: torch.Tensor, tok_seq: torch.Tensor, tok_pos: torch.Tensor, *, n_head: int,
                     scale: float, window: int = 0, n_splits: int = 1, partials: Optional[torch.Tensor] = None,
                     tok_list: Optional[torch.Tensor] = None, n_tokens: Optional[int] = None, waves: int = 4,
                     rows_are_requests: bool = False, leave_splits: bool = False, chunk: int = 0,
                     num_pages: Optional[int] = None) -> None:
    """Each token on its own over its request's cache (bfloat16, or float32 throughout), its keys cut into `n_splits`.
    With `tok_list` (int32) only those rows are computed. `rows_are_requests`: row t belongs to
    request t (every request brings one token), which saves the kernel a lookup. With
    `leave_splits` (several splits) `out` is not written: `partials`, viewed as [tokens, heads,
    splits, head size + 4], keeps each split's weighted values, maximum and sum for a reader
    that merges them (`gemm_att_parts`). `chunk` > 0: split z takes keys [z * chunk, (z + 1) * chunk) of a
    token's keys instead of an equal share (`n_splits * chunk` must cover the longest context): a token's
    sums then follow from its position alone."""
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
    _, hkv, page, hd = k_cache.shape
    os_, qs = _rows(out, "out"), _rows(q, "q")
    rows = out.shape[0]
    n = rows if n_tokens is None else n_tokens
    if q.shape[0] != rows or q.shape[1] < n_head * hd or out.shape[1] != n_head * hd:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {n_head} heads of {hd}")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype) or q.dtype not in (torch.bfloat16, torch.float32):
        raise KernelError("attention_decode: q, out and the caches must all be bfloat16 or all float32")
    _dev(block_tables, "block_tables")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise KernelError("attention: block_tables must be contiguous int32 [requests, max_blocks]")
    _i32(tok_seq, "tok_seq", rows)
    _i32(tok_pos, "tok_pos", rows)
    if tok_list is not None:
        _i32(tok_list, "tok_list", n)
    elif n != rows:
        raise KernelError("attention_decode: n_tokens needs tok_list")
    if leave_splits and n_splits <= 1:
        raise KernelError("attention_decode: splits are left only when there are several")
    if n_splits > 1:
        need = n * n_head * n_splits * (hd + 4)
        if partials is None or partials.dtype != torch.float32 or partials.numel() < need or not partials.is_contiguous():
            raise KernelError(f"attention_decode: {n_splits} splits need {need} float32 of partials")
    _lib.call("liyab_attention_decode", out.data_ptr(), os_, q.data_ptr(), qs, k_cache.data_ptr(), v_cache.data_ptr(),
              dtype_code(q.dtype), block_tables.data_ptr(), block_tables.shape[1], _ptr(tok_list), tok_seq.data_ptr(), tok_pos.data_ptr(),
              n, float(scale), int(window), n_head, hkv, hd, page, n_splits, int(chunk), waves, 1 if rows_are_requests else 0,
              _ptr(partials), 1 if leave_splits else 0, _pages(k_cache, num_pages), _stream())


def attention_merge(out: torch.Tensor, partials: torch.Tensor) -> None:
    """out [tokens, heads * head size] (bfloat16 or float32) = the splits that `attention_decode(...,
    leave_splits=True)` left in partials [tokens, heads, splits, head size + 4], merged in split order."""
    _dev(partials, "partials")
    os_ = _rows(out, "out")
    if partials.dtype != torch.float32 or partials.dim() != 4 or not partials.is_contiguous():
        raise KernelError("attention_merge: partials must be contiguous float32 [tokens, heads, splits, head size + 4]")
    n, H, S, hd4 = partials.shape
    if out.dtype not in (torch.bfloat16, torch.float32) or tuple(out.shape) != (n, H * (hd4 - 4)):
        raise KernelError(f"attention_merge: out must be bfloat16 or float32 [{n}, {H * (hd4 - 4)}]")
    _lib.call("liyab_attention_merge", out.data_ptr(), dtype_code(out.dtype), os_, partials.data_ptr(), n, H, hd4 - 4, S, _stream())


def attention_prefill(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      block_tables: torch.Tensor, work: torch.Tensor, n_tiles: int, *, n_head: int, scale: float,
                      window: int = 0, tile: int = 128, ksplit: int = 1, num_pages: Optional[int] = None) -> None:
    """Tiles of up to `tile` (64 or 128) consecutive queries of one request over its bfloat16
    cache, on the matrix cores; `ksplit` waves (1, 2, or 4 with tiles of 64) share the keys of
    32 queries. work: int32 [n_tiles, 4] = (request index, first row, first
    position, queries); the caller has checked rows and positions against out and the block tables."""
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise KernelError("attention: caches must be contiguous [pages, kv_heads, page_size, head_dim] of one shape")
    _, hkv, page, hd = k_cache.shape
    os_, qs = _rows(out, "out"), _rows(q, "q")
    if q.shape[0] != out.shape[0] or q.shape[1] < n_head * hd or out.shape[1] != n_head * hd:
        raise KernelError(f"attention: q {tuple(q.shape)} / out {tuple(out.shape)} do not fit {n_head} heads of {hd}")
    if not (q.dtype == out.dtype == k_cache.dtype == v_cache.dtype == torch.bfloat16):
        raise KernelError("attention_prefill: q, out and the caches must be bfloat16")
    if not prefill_takes(hd):
        raise KernelError(f"attention_prefill: head size {hd} is not a multiple of 16 in 16..128")
    _dev(block_tables, "block_tables")
    if block_tables.dim() != 2 or block_tables.dtype != torch.int32 or not block_tables.is_contiguous():
        raise KernelError("attention: block_tables must be contiguous int32 [requests, max_blocks]")
    _i32(work, "work", 4 * n_tiles)
    _lib.call("liyab_attention_prefill", out.data_ptr(), os_, q.data_ptr(), qs, k_cache.data_ptr(), v_cache.data_ptr(),
              block_tables.data_ptr(), block_tables.shape[1], work.data_ptr(), n_tiles, int(tile), int(ksplit), float(scale), int(window),
              n_head, hkv, hd, page, _pages(k_cache, num_pages), _stream())


PREFILL_KSPLIT4_WORK = 256  # tiles x heads up to which four waves share a tile of 64 queries' keys


def prefill_takes(hd: int) -> bool:
    return hd % 16 == 0 and 16 <= hd <= 128


def decode_plan(n_tokens: int, n_head: int, context_bucket: int):
    """(splits of the keys, waves per workgroup) for tokens whose attention the kernel finishes
    itself (several splits: plus the merge kernel). `context_bucket`: the most keys a token has,
    rounded up. From measurements at 12 to 32 heads of 64 and 128, 1 to 8 tokens and 300 to
    4,000 keys (us, attention and merge): with many (token, head) pairs a workgroup of 4 waves
    a pair is fastest, with a few hundred one of 8 (a decode step at batch 24 / 32 / 40 with 4,
    8 and 16 waves: 610 595 654 / 648 633 692 / 706 698 755; 200 pairs at 544 / 2,000 keys: 7.1
    / 19.7 with 8 waves, 8.9 / 20.0 with 16). With fewer pairs than would fill the chip the keys
    are cut across workgroups of 4 waves, into 4, 8 or 16 splits of 128 keys or more, while
    pairs x splits stay within the chip's 256 compute units (32 pairs of 128 dimensions at
    1,000 / 2,000 / 4,000 keys: 7.5 / 10.6 / 18.4 in 8 splits against 11.8 / 19.1 / 33.1 uncut
    on 16 waves; 12 pairs of 64: 6.9 / 7.8 / 9.7 against 8.7 / 11.8 / 18.6). Two splits never
    beat 8 waves uncut. Uncut, 16 waves a pair pay from 4,000 keys on only."""
    pairs = max(1, n_tokens * n_head)
    if pairs >= 512 or context_bucket <= 256:
        return 1, 4
    splits = 1
    while splits < 16 and pairs * splits * 2 <= 256 and context_bucket // (splits * 2) >= 128:
        splits *= 2
    if splits >= 4:
        # (splits of 1,024 keys and more on 8 waves: 12 pairs at 30,000 keys in 16 splits 26.7 us on
        # 4 waves, 22.4 on 8; 32 pairs of 128 dimensions 92.6 and 89.1)
        return splits, (8 if context_bucket // splits >= 1024 else 4)
    return 1, (16 if context_bucket >= 4096 and pairs < 256 else 8)


def decode_split_plan(n_tokens: int, n_head: int, context_bucket: int):
    """(splits, waves per workgroup) for a step whose attention output is read by somebody who
    merges a (token, head) pair's splits himself (1 split: not cut). Measured at 12 heads of 64
    and contexts of 512 to 1,024 (us a decode step at batch 1 / 8 / 16, uncut: 376 / 430 / 499):
    8 splits of 4 waves 347 / 418 / 505, 4 of 4 360 / 425 / 496, 4 of 8 353 / 426 / 503, 2 of
    16 390 / 444 / 588. So: workgroups of 4 waves, 8 splits (4 from a hundred pairs on), a
    split keeping 128 keys or more of the longest context."""
    pairs = max(1, n_tokens * n_head)
    most = 8 if pairs <= 96 else (4 if pairs <= SPLIT4_PAIRS else (2 if pairs <= SPLIT2_PAIRS else 1))
    splits = 1
    while splits < most and context_bucket // (2 * splits) >= 128:
        splits *= 2
    # very long contexts of one or two requests: 8 splits of 4 waves leave most of the chip idle and
    # each walks thousands of keys; 16 waves a split walk them four times as fast (us, 12 pairs of 64
    # at 8,000 / 16,000 / 30,000 keys: 14.5 / 25.1 / 41.2 on 4 waves, 11.7 / 17.0 / 23.6 on 16; from
    # 48 pairs on 4 waves win)
    return splits, (16 if pairs <= 32 and context_bucket // splits >= 1024 else 4)


# pairs up to which 4 and 2 splits are taken (beyond 16 tokens splits lost: us a step at batch 17 / 24 / 32
# uncut 529 / 594 / 633, in 4 splits 568 / 630 / 708, in 2 splits 573 / 635 / 704)
SPLIT4_PAIRS, SPLIT2_PAIRS = 192, 192


ATTENTION_MAX_HEAD_DIM = 256  # what the attention kernels take (attention_generic.hip, attention_decode.hip)


INVARIANT_CHUNK = 256  # keys a split where splits go by position alone
INVARIANT_SPLIT_WORK = 1024  # (token, head, split) workgroups up to which such splits are launched side by side
INVARIANT_MAX_SPLITS = 16  # what one workgroup walks in turn (attention_decode.hip: AD_LOOP_CHUNKS)


def invariant_chunk(reach: int) -> int:
    """Keys a split where splits go by position alone, for requests that reach at most `reach` keys:
    INVARIANT_CHUNK, doubled until INVARIANT_MAX_SPLITS splits cover the reach."""
    chunk = INVARIANT_CHUNK
    while chunk * INVARIANT_MAX_SPLITS < reach:
        chunk *= 2
    return chunk


def attention_takes(head_dim: int) -> bool:
    """Whether some attention kernel of the library takes this head size, in either precision."""
    return 0 < head_dim <= ATTENTION_MAX_HEAD_DIM


def attention(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
              block_tables: torch.Tensor, ctx, *, n_head: int, scale: float, window: int = 0,
              splits_ok: bool = False) -> Optional[torch.Tensor]:
    """Attention of the step's tokens over their requests' cached keys and values; the kernel
    is chosen from the step's shape (`ctx` is the step's StepContext; `ctx.plans["attention"]`
    says how the step's tokens are cut, see parts/attention.py; without it every token goes to
    the plain kernel). With `splits_ok`, a step of few tokens may leave `out` unwritten and
    return the splits of each (token, head) pair instead, float32 [tokens, heads, splits, head
    size + 4], for `gemm_att_parts`."""
    hd = k_cache.shape[3]
    host = ctx.host
    plan = ctx.plans.get("attention")
    fast = (plan is not None and q.dtype == torch.bfloat16 and hd % 8 == 0 and q.stride(0) % 8 == 0
            and out.stride(0) % 8 == 0)

    def decode(tok_list, n):
        splits, waves = decode_plan(n, n_head, min(plan.context_bucket, window) if window > 0 else plan.context_bucket)
        partials = None
        if splits > 1:
            partials = ctx.workspace.get("attn_partials", (n * n_head * splits * (hd + 4),), torch.float32)
        attention_decode(out, q, k_cache, v_cache, block_tables, ctx.tok_seq, ctx.positions, n_head=n_head,
                         scale=scale, window=window, n_splits=splits, partials=partials, waves=waves,
                         tok_list=tok_list, n_tokens=n if tok_list is not None else None,
                         rows_are_requests=tok_list is None and host.max_q_len == 1)

    if (plan is not None and block_tables.shape[1] <= 2048
            and (fast and _invariant or q.dtype == torch.float32 and hd % 8 == 0 and q.stride(0) % 4 == 0 and out.stride(0) % 4 == 0)):
        # the 32-bit path and the batch-invariant mode: every token on its own on four waves, its keys
        # in splits of INVARIANT_CHUNK from its first key on, merged in their order: the order of a
        # token's sums follows from its position alone, so its bits do not depend on the batch
        n = out.shape[0]
        # a split's keys follow from what a request can reach at most (the table's width, the window): a
        # constant of the engine, never of the step; at most 16 splits, so that one workgroup can walk them
        # all and the merge's arrays hold them (contexts past 4,096 keys take longer splits)
        reach = block_tables.shape[1] * k_cache.shape[2] if window <= 0 else min(window, block_tables.shape[1] * k_cache.shape[2])
        chunk = invariant_chunk(reach)
        splits = max(1, -(-min(plan.context_bucket, reach) // chunk))
        # many tokens: a workgroup walks its token's splits in turn (the same bits: the kernel merges them
        # as the merge kernel does), which saves the splits' traffic and leaves the chip as full
        if n * n_head * splits > INVARIANT_SPLIT_WORK:
            splits = 1
        partials = ctx.workspace.get("attn_partials", (n * n_head * splits * (hd + 4),), torch.float32) if splits > 1 else None
        attention_decode(out, q, k_cache, v_cache, block_tables, ctx.tok_seq, ctx.positions, n_head=n_head, scale=scale,
                         window=window, n_splits=splits, partials=partials, waves=4, chunk=chunk,
                         rows_are_requests=host.max_q_len == 1)
        return None
    if fast and plan.mode == "decode" and block_tables.shape[1] <= 2048:
        n = out.shape[0]
        splits, waves = decode_split_plan(n, n_head, plan.context_bucket) if splits_ok else (1, 4)
        if splits > 1 and att_parts_takes(n, splits, hd):
            partials = ctx.workspace.get("attn_partials", (n, n_head, splits, hd + 4), torch.float32)
            attention_decode(out, q, k_cache, v_cache, block_tables, ctx.tok_seq, ctx.positions, n_head=n_head,
                             scale=scale, window=window, n_splits=splits, partials=partials, waves=waves,
                             rows_are_requests=host.max_q_len == 1, leave_splits=True)
            return partials
        decode(None, n)
        return None
    if fast and plan.mode == "prefill" and prefill_takes(hd) and scale > 0 and block_tables.shape[1] <= 2048:
        # long portions in tiles on the matrix cores, the short ones token by token
        if plan.n_tiles:
            # with fewer workgroups than compute units, two waves share each query group's keys:
            # the longest tile's walk over its keys is then the kernel's critical path, and halves
            work = plan.n_tiles * n_head
            # (heads past 96: two waves a query group at every size, 185 against 217 us for 16 x 1,024 tokens of 12 heads of 128)
            ksplit = (4 if plan.tile == 64 and hd <= 64 and work <= PREFILL_KSPLIT4_WORK else 2) if work <= 256 or hd > 96 else 1
            attention_prefill(out, q, k_cache, v_cache, block_tables, plan.work, plan.n_tiles, n_head=n_head,
                              scale=scale, window=window, tile=plan.tile, ksplit=ksplit)
        if plan.n_single:
            decode(plan.single_rows, plan.n_single)
        return
    attention_generic(out, q, k_cache, v_cache, block_tables, ctx.tok_seq, ctx.positions, n_head=n_head, scale=scale,
                      window=window)
