"""Matrix products of the parts: y = x . W^T (+ bias) with an epilogue.

W is [out, in], a row per output feature, the layout the reference works in
(include/liyab/types.h:165-184; y = x . W^T, include/liyab/backend.h:35).
The kernel is chosen here by dtype and shape; callers only say what they
want computed. The first operand may be a pending norm (`Normed`): the norm
runs first as its own kernel, unless FOLD_NORM asks for the product kernel
that applies the norm itself where the shape allows it.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .norms import Normed


# Folding the norm into a decode step's products saves a launch, but every workgroup of the
# product then repeats the norm ahead of its multiplies. Measured at GPT-2 small's sizes the
# standalone norm (a wave per row, 2.6 us) plus the plain product is faster: 464 against 506 us
# a step at batch 1, 526 against 574 at batch 8. Off; the folded kernel stays available.
FOLD_NORM = False


def _fuses(a, w: torch.Tensor) -> bool:
    return (FOLD_NORM and isinstance(a, Normed) and getattr(a.norm, "fusable", None) == "layernorm" and w.dtype == torch.bfloat16
            and a.x.dtype == torch.float32 and a.x.is_contiguous() and ops.skinny_ln_takes(a.n_rows, a.norm.width, w.shape[0]))


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
    if _fuses(a, w):
        n = a.norm
        ops.gemm_skinny_ln(a.x, n.weight, n.bias, n.eps, w, bias, rows=a.rows, n_rows=a.n_rows, out=out,
                           residual=residual, epilogue=epilogue, kv=kv)
        return
    if isinstance(a, Normed):
        a = a.tensor()
    ops.gemm(a, w, bias, out=out, residual=residual, epilogue=epilogue, kv=kv)


def linear_deferred(a, w: torch.Tensor, bias: Optional[torch.Tensor], ctx, name: str):
    """a . w^T + bias as sums still to be added to the residual stream, or None where the
    product is not worth cutting over its inner dimension (the caller then adds it through
    `linear(..., residual=)`). The planes live in the step's workspace under `name` until the
    next reader of the stream has added them."""
    from .base import PendingSums

    a = a.tensor() if isinstance(a, Normed) else a
    if a.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or a.shape[0] > 64:
        return None
    parts = ops.k_parts(a.shape[0], w.shape[0], a.shape[1])
    if parts <= 1:
        return None
    planes = ctx.workspace.get(name, (parts, a.shape[0], w.shape[0]), torch.float32)
    ops.gemm_skinny_parts(a, w, planes)
    return PendingSums(planes, bias)


def paged_qkv_takes(dtype: torch.dtype, k: int) -> bool:
    """Whether the product kernels for this dtype and inner size can write keys and values
    into cache pages from their epilogue."""
    return dtype == torch.bfloat16 and k % 8 == 0
