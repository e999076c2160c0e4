"""y = x W^T for a weight stored [out, in] (the orientation a checkpoint stores
a linear layer in; reference: engine/include/llm/kernels.h:48-57), and the
choice of kernel for it (reference: matmul dispatch, engine/src/model.cpp:153-192):
up to 64 rows the weight-streaming kernel (with RMSNorm fused in up to 16 rows),
beyond that the tiled matrix-core kernel, and the plain float kernel for
everything those refuse (float32 operands, k no multiple of 8)."""
from __future__ import annotations

from typing import Optional, Union

import torch

from ..csrc import ops
from .lazy import Normed


def _fused_norm(x: Normed, w, epilogue: int) -> Optional[torch.Tensor]:
    if x._tensor is not None:
        return None
    scale = x.fusable_scale()
    if scale is None or not ops.gemm_normed_supported(x.x, x.n_rows, scale[0], w):
        return None
    return ops.gemm_normed(x.x, x.rows, x.n_rows, scale[0], scale[1], w, epilogue)


def _prepared_norm(x: Normed, w, epilogue: int) -> Optional[torch.Tensor]:
    """The product from what the product before left for this norm, where there is such a thing."""
    if x.pre is None or x._tensor is not None or not ops.gemm_prenormed_supported(x.pre, w, epilogue):
        return None
    return ops.gemm_prenormed(x.pre, w, epilogue)


def linear(x: Union[torch.Tensor, Normed], w, out_dtype: Optional[torch.dtype] = None,
           accumulate_into: Optional[torch.Tensor] = None, ctx=None) -> torch.Tensor:
    """x [M, K] times w [N, K] transposed (w a tensor or an ops.StreamedWeight).  With
    ``accumulate_into`` (the float32 residual stream) the product is added to it in place; with
    ``ctx`` too, and a norm named as the next reader of the stream (``ctx.handoff.reading_next``), the
    product prepares that norm where its kernel can and leaves the result with the handoff: the norm
    itself (ops.Finished) where the product cuts k over workgroups anyway -- the kernel that adds the parts
    up norms the stream on its way, which serves every reader -- or else, if the reader takes that, the parts
    of the norm that a product can finish (ops.Prenormed)."""
    if isinstance(x, Normed):
        if accumulate_into is None and out_dtype in (torch.bfloat16, torch.float32):
            epi = ops.EPI_STORE_BF16 if out_dtype == torch.bfloat16 else ops.EPI_STORE_F32
            fused = _prepared_norm(x, w, epi)
            if fused is None:
                fused = _fused_norm(x, w, epi)
            if fused is not None:
                return fused
        x = x.tensor()
    reading = ctx.handoff.reading_next if ctx is not None and accumulate_into is not None else None
    if reading is not None:
        norm, takes_parts = reading
        scale = norm.fusable() if hasattr(norm, "fusable") else None
        if scale is not None and ops.gemm_parts_supported(x, w, accumulate_into, scale[0]):
            ctx.handoff.leave(norm, ops.gemm_parts_accumulate_norm(x, w, accumulate_into, scale[0], scale[1], checked=True))
            return accumulate_into
        if scale is not None and takes_parts and ops.gemm_emit_supported(x, w, accumulate_into, scale[0]):
            ctx.handoff.leave(norm, ops.gemm_accumulate_emit(x, w, accumulate_into, scale[0], scale[1]))
            return accumulate_into
    fast = ops.gemm_fast(x, w, out_dtype, accumulate_into)
    if fast is not None:
        return fast
    return ops.gemm_generic(x, w, out_dtype, accumulate_into)


def linear_swiglu(x: Union[torch.Tensor, Normed], w_gate_up, interleaved: bool = False) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) for w_gate_up = gate rows followed by up rows, or (interleaved)
    blocks of eight gate rows and the eight up rows of the same outputs."""
    if isinstance(x, Normed):
        fused = None
        if interleaved and w_gate_up.shape[0] % 16 == 0:
            fused = _prepared_norm(x, w_gate_up, ops.EPI_SWIGLU)
            if fused is None:
                fused = _fused_norm(x, w_gate_up, ops.EPI_SWIGLU)
        if fused is not None:
            return fused
        x = x.tensor()
    return ops.gemm_swiglu(x, w_gate_up, interleaved)
