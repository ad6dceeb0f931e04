"""Un-normalised bidirectional linear attention (drop-in for
flash_bla/ops/simple_la/fused.py:495-656):  o = q (scale * K^T V)."""
from typing import Optional

import torch

from flash_bla import _hip
from flash_bla.ops._check import check_dense
from flash_bla.ops.feature_map import applied_on_load, check_feature_map, elu_plus_one, mapped_in_kernels
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


class MappedSimpleLinearAttnFunction(torch.autograd.Function):
    """simple_la(elu(q) + 1, elu(k) + 1, v) as one autograd node (16-bit heads of 64 x 64): forward
    and backward kernels map q and k as they load them, dq and dk come back with respect to the
    raw tensors (see MappedLinearAttnFunction in ops/linear_attn/fused.py)."""

    @staticmethod
    @contiguous
    def forward(ctx, q, k, v, scale):
        o, s, _ = _hip.la_fwd(q, k, v, None, None, scale, 0.0, _hip.ELU1_QK)
        ctx.save_for_backward(q, k, v, s)
        ctx.scale = scale
        return o

    @staticmethod
    @contiguous
    def backward(ctx, do):
        q, k, v, s = ctx.saved_tensors
        dq, dk, dv, _, _ = _hip.la_bwd(q, k, v, None, None, do, s, None, ctx.scale, 0.0,
                                       _hip.ELU1_QK | _hip.ELU1_GRAD)
        return dq, dk, dv, None


def simple_la(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    retuen_states: Optional[bool] = False,
    feature_map: Optional[str] = None,
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
        feature_map: None (the reference's signature) or "elu+1": q and k are given before the
            feature map `elu(x) + 1`, which the kernels of 16-bit heads of 64 x 64 apply as they
            load them (forward and backward); other shapes map first with one launch.
    """
    check_dense("simple_la", q, k, v)
    if scale is None:
        scale = q.shape[-1] ** -0.5
    if check_feature_map(feature_map):
        if applied_on_load(q, k, v):
            return _hip.la_fwd(q.contiguous(), k.contiguous(), v.contiguous(), None, None, scale, 0.0,
                               _hip.ELU1_QK)[0]
        if mapped_in_kernels(q, v):
            return MappedSimpleLinearAttnFunction.apply(q, k, v, scale)
        q, k = elu_plus_one(q, k)
    return SimpleLinearAttnFunction.apply(q, k, v, scale)
