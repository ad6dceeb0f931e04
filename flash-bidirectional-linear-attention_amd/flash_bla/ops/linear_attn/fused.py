"""Normalised bidirectional linear attention (drop-in for
flash_bla/ops/linear_attn/fused.py:350-480).

    S = scale * K^T V,  km = mean_t k_t,  o_t = (q_t S) / (q_t . km + eps)

The forward and backward launch hand-written gfx950 kernels through
libfbla_hip.so.  The state (S, km) is kept in fp32 and saved for the backward,
which recomputes o.dO from q and S instead of re-reading o.
"""
from typing import Optional

import torch

from flash_bla import _hip
from flash_bla.ops._check import check_dense
from flash_bla.ops.feature_map import applied_on_load, check_feature_map, elu_plus_one, mapped_in_kernels
from flash_bla.utils import contiguous


class LinearAttnFunction(torch.autograd.Function):
    """Counterpart of LinearAttnFunction (linear_attn/fused.py:350-453)."""

    @staticmethod
    @contiguous
    def forward(ctx, q, k, v, scale, eps):
        o, s, km = _hip.la_fwd(q, k, v, None, None, scale, eps, _hip.NORMALIZE)
        ctx.save_for_backward(q, k, v, s, km)
        ctx.scale = scale
        ctx.eps = eps
        return o

    @staticmethod
    @contiguous
    def backward(ctx, do):
        q, k, v, s, km = ctx.saved_tensors
        dq, dk, dv, _, _ = _hip.la_bwd(q, k, v, None, None, do, s, km, ctx.scale, ctx.eps,
                                       _hip.NORMALIZE)
        return dq, dk, dv, None, None


class MappedLinearAttnFunction(torch.autograd.Function):
    """linear_attention(elu(q) + 1, elu(k) + 1, v) as one autograd node (16-bit heads of 64 x 64).
    No mapped copy of q or k is ever written: the forward kernels map q and k as they load them,
    the backward kernels do the same and return dq and dk with respect to the raw tensors (times
    min(mapped, 1), the map's derivative), so the map costs no launch and no tensor pass of its
    own in either direction."""

    @staticmethod
    @contiguous
    def forward(ctx, q, k, v, scale, eps):
        o, s, km = _hip.la_fwd(q, k, v, None, None, scale, eps, _hip.NORMALIZE | _hip.ELU1_QK)
        ctx.save_for_backward(q, k, v, s, km)
        ctx.scale = scale
        ctx.eps = eps
        return o

    @staticmethod
    @contiguous
    def backward(ctx, do):
        q, k, v, s, km = ctx.saved_tensors
        dq, dk, dv, _, _ = _hip.la_bwd(q, k, v, None, None, do, s, km, ctx.scale, ctx.eps,
                                       _hip.NORMALIZE | _hip.ELU1_QK | _hip.ELU1_GRAD)
        return dq, dk, dv, None, None


def linear_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    eps: float = 1e-6,
    feature_map: Optional[str] = None,
) -> torch.Tensor:
    r"""
    Args:
        q: queries of shape `(B, H, L, K)` (positive features, e.g. elu+1)
        k: keys of shape `(B, H, L, K)`
        v: values of shape `(B, H, L, V)`
        scale: factor applied to the key-value state; defaults to `1 / L`
            (linear_attn/fused.py:477-478).
        eps: constant added to the denominator.
        feature_map: None (the reference's signature: q and k are features already) or "elu+1":
            q and k are given before the blocks' feature map `elu(x) + 1`
            (layers/linfusion.py:88-89).  An inference forward of 16-bit heads of 64 x 64 applies
            it inside the kernels as they load q and k (no mapped copies are written); with
            gradients, the backward kernels of the same heads map q and k on load as well and
            return dq, dk with respect to the raw tensors; every other call maps them first and
            lets autograd differentiate the map.
    Returns the output of shape `(B, H, L, V)` with `v`'s dtype.
    """
    check_dense("linear_attention", q, k, v)
    if scale is None:
        scale = k.shape[-2] ** -1.0
    if check_feature_map(feature_map):
        if applied_on_load(q, k, v):
            return _hip.la_fwd(q.contiguous(), k.contiguous(), v.contiguous(), None, None, scale, eps,
                               _hip.NORMALIZE | _hip.ELU1_QK)[0]
        if mapped_in_kernels(q, v):
            return MappedLinearAttnFunction.apply(q, k, v, scale, eps)
        q, k = elu_plus_one(q, k)
    return LinearAttnFunction.apply(q, k, v, scale, eps)
