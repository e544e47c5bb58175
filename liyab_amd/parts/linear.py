"""Matrix products of the parts: y = x . W^T (+ bias) with an epilogue.

W is [out, in], a row per output feature, the layout the reference works in
(include/liyab/types.h:165-184; y = x . W^T, include/liyab/backend.h:35).
The kernel is chosen here by dtype and shape; callers only say what they
want computed.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops


def linear(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], *, out: Optional[torch.Tensor] = None,
           residual: Optional[torch.Tensor] = None, activation: str = "none") -> None:
    """out = act(a . w^T + bias), or with `residual` given: residual += a . w^T + bias."""
    if residual is not None:
        ops.gemm(a, w, bias, residual=residual, epilogue=ops.EPI_RESIDUAL)
    else:
        ops.gemm(a, w, bias, out=out, epilogue=ops.ACTIVATION_EPILOGUE[activation])
