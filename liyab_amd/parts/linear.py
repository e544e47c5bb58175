"""Matrix products of the parts: y = x . W^T (+ bias) with an epilogue.

W is [out, in], a row per output feature, the layout the reference works in
(include/liyab/types.h:165-184; y = x . W^T, include/liyab/backend.h:35).
The kernel is chosen here by dtype and shape; callers only say what they
want computed. The first operand may be a pending norm (`Normed`): where the
shape allows it the product kernel applies the norm itself (FOLD_NORM),
otherwise the norm runs first as its own kernel.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .norms import Normed


# Folding the norm into a decode step's products saves a launch of the seven a layer has; every
# workgroup of the product then repeats the norm of all rows ahead of its multiplies, which
# pays while the rows are few (us a decode step at GPT-2 small's sizes, folded and not: 8 rows
# 420 / 471, 16 rows 498 / 524, 24 rows 657 / 679, 32 rows 711 / 694, 64 rows 954 / 810; and 64 rows
# with a workgroup normalising 32 of them for 32 output features, a wave asking for its four rows
# together, where the stream is whole (the feed-forward's first product): 721 against 713, 48 rows 656
# against 652. That form was taken out again.)
FOLD_NORM = True
FOLD_NORM_ROWS = 24
TILED_PARTS = True  # products of 33 to 64 rows that are added to the stream: tiled and cut over K (ops.tiled_k_parts)


def _fuses(a, w: torch.Tensor, residual) -> bool:
    return (FOLD_NORM and isinstance(a, Normed) and getattr(a.norm, "fusable", None) == "layernorm" and residual is None
            and a.rows is None and a._tensor is None and w.dtype == torch.bfloat16 and a.x.dtype == torch.float32
            and a.x.is_contiguous() and a.n_rows <= FOLD_NORM_ROWS
            and ops.skinny_ln_pays(a.n_rows, w.shape[0], a.norm.width))


def linear(a, w: torch.Tensor, bias: Optional[torch.Tensor], *, out: Optional[torch.Tensor] = None,
           residual: Optional[torch.Tensor] = None, activation: str = "none", kv=None) -> None:
    """out = act(a . w^T + bias); with `residual`: residual += a . w^T + bias; with `kv` =
    (k_cache, v_cache, slots, q_dim): queries to `out`, keys and values into their pages."""
    if residual is not None:
        epilogue = ops.EPI_RESIDUAL
    elif kv is not None:
        epilogue = ops.EPI_QKV_PAGED
    else:
        epilogue = ops.ACTIVATION_EPILOGUE[activation]
    if _fuses(a, w, residual):
        n = a.norm
        ops.gemm_skinny_ln(a.x, n.weight, n.bias, n.eps, w, bias, out=out, epilogue=epilogue, kv=kv)
        return
    if isinstance(a, Normed):
        a = a.tensor()
    ops.gemm(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv)


def _overlap(a: torch.Tensor, b: torch.Tensor) -> bool:
    a0, b0 = a.data_ptr(), b.data_ptr()
    return a0 < b0 + b.numel() * b.element_size() and b0 < a0 + a.numel() * a.element_size()


def linear_deferred(a, w: torch.Tensor, bias: Optional[torch.Tensor], ctx, name: str, stream):
    """stream + a . w^T + bias as a split residual stream (`a` may be attention's output still
    in splits, float32 [tokens, heads, splits, head size + 4]), or None where the product is not
    worth cutting over its inner dimension (the caller then adds it through `linear(...,
    residual=settled(stream))`). `stream` is the residual stream the product is added to, a
    tensor or a SplitStream; the planes live in the step's workspace under `name` until the
    next product cut this way writes its own under another name."""
    from .base import SplitStream

    if ops.is_batch_invariant():
        return None  # no cut over K: its parts would follow the step's size
    a = a.tensor() if isinstance(a, Normed) else a
    in_splits = a.dim() == 4  # attention's output as its splits [tokens, heads, splits, head size + 4]
    M, K = (a.shape[0], a.shape[1] * (a.shape[3] - 4)) if in_splits else a.shape
    if (a.dtype != torch.bfloat16 and not in_splits) or w.dtype != torch.bfloat16:
        return None
    parts = ops.k_parts(M, w.shape[0], K)
    tiled = False
    if parts <= 1 and not in_splits and TILED_PARTS:
        parts = ops.tiled_k_parts(M, w.shape[0], K)  # one tile of 33 to 64 rows: the tiled kernel, cut over K
        tiled = parts > 1
    split = isinstance(stream, SplitStream)
    if parts <= 1:
        # not worth cutting; but a stream that arrives split is taken as it is by the streaming
        # kernel's epilogue (one plane written: the sum of the stream's planes, the bias and the
        # product), where settling it first would be a kernel of its own
        if not (split and not in_splits and ops.skinny_parts_takes(M, w.shape[0], K)):
            return None
        parts = 1
    base = stream.planes if split else stream
    planes = ctx.workspace.get(name, (parts, M, w.shape[0]), torch.float32)
    if _overlap(planes, base):
        return None  # the stream's planes are where these would go
    if in_splits:
        ops.gemm_att_parts(a, w, planes, bias=bias, base=base)
    elif tiled:
        # 64 x 32 tiles while every tile of every part has a compute unit of its own (128 rows,
        # 3,072 -> 768 in four parts: 6.5 against 7.5 us in 64 x 64 tiles), 64 x 64 tiles beyond
        few = (M + 63) // 64 * ((w.shape[0] + 31) // 32) * parts <= ops.compute_units()
        fewer = (M + 31) // 32 * ((w.shape[0] + 31) // 32) * parts <= ops.compute_units()  # 32 x 32 tiles each on a compute unit of its own
        if M <= 64 and w.shape[0] > 2048:  # one tile of rows, many output features: the largest tile that takes the rows (ops.tiled_k_parts)
            tile = 17 if M <= 32 else 6
        else:
            tile = 17 if fewer else (16 if M <= 64 or few else 6)
        ops.gemm_mfma_dl_parts(a, w, planes, bias=bias, base=base, tile=tile)
    else:
        ops.gemm_skinny_parts(a, w, planes, bias=bias, base=base)
    return SplitStream(planes, stream.home if split else stream)


def paged_qkv_takes(dtype: torch.dtype, k: int) -> bool:
    """Whether the product kernels for this dtype and inner size can write keys and values
    into cache pages from their epilogue."""
    return dtype == torch.bfloat16 and k % 8 == 0
