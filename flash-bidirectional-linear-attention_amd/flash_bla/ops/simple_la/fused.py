"""Un-normalised bidirectional linear attention (drop-in for
flash_bla/ops/simple_la/fused.py:495-656):  o = q (scale * K^T V)."""
from typing import Optional

import torch

from flash_bla import _hip
from flash_bla.ops._check import check_dense
from flash_bla.utils import contiguous


class SimpleLinearAttnFunction(torch.autograd.Function):
    """Counterpart of SimpleLinearAttnFunction (simple_la/fused.py:495-626)."""

    @staticmethod
    @contiguous
    def forward(ctx, q, k, v, scale):
        o, s, _ = _hip.la_fwd(q, k, v, None, None, scale, 0.0, 0)
        ctx.save_for_backward(q, k, v, s)
        ctx.scale = scale
        return o

    @staticmethod
    @contiguous
    def backward(ctx, do):
        q, k, v, s = ctx.saved_tensors
        dq, dk, dv, _, _ = _hip.la_bwd(q, k, v, None, None, do, s, None, ctx.scale, 0.0, 0)
        return dq, dk, dv, None


def simple_la(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    retuen_states: Optional[bool] = False
) -> torch.Tensor:
    r"""
    Args:
        q: queries of shape `(B, H, L, K)`
        k: keys of shape `(B, H, L, K)`
        v: values of shape `(B, H, L, V)`
        scale: factor applied to the key-value state; defaults to `K ** -0.5`
            (simple_la/fused.py:648-649).
        retuen_states: accepted and ignored, as in the reference
            (simple_la/fused.py:634,653-654).
    """
    check_dense("simple_la", q, k, v)
    if scale is None:
        scale = q.shape[-1] ** -0.5
    return SimpleLinearAttnFunction.apply(q, k, v, scale)
