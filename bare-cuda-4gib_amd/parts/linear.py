"""y = x W^T for a weight stored [out, in] (the orientation a checkpoint stores
a linear layer in; reference: engine/include/llm/kernels.h:48-57), and the
choice of kernel for it (reference: matmul dispatch, engine/src/model.cpp:153-192)."""
from __future__ import annotations

from typing import Optional

import torch

from ..csrc import ops


def linear(x: torch.Tensor, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           accumulate_into: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [M, K] times w [N, K] transposed.  With ``accumulate_into`` (the
    float32 residual stream) the product is added to it in place."""
    fast = ops.gemm_fast(x, w, out_dtype, accumulate_into)
    if fast is not None:
        return fast
    return ops.gemm_generic(x, w, out_dtype, accumulate_into)
