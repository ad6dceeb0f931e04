"""Decoupled bidirectional linear attention (drop-in for
flash_bla/ops/linear_attn/decoupled.py:411-542): the numerator uses the rotary
features, the denominator the plain ones.

    S = scale * K_rope^T V,  km = mean_t k_t,  o_t = (q_rope_t S) / (q_t . km + eps)
"""
from typing import Optional

import torch

from flash_bla import _hip
from flash_bla.ops._check import check_dense
from flash_bla.utils import contiguous

_FLAGS = _hip.NORMALIZE | _hip.DECOUPLED


class DecoupledLAFunction(torch.autograd.Function):
    """Counterpart of DecoupledLAFunction (decoupled.py:411-509)."""

    @staticmethod
    @contiguous
    def forward(ctx, q, k, q_rope, k_rope, v, scale, eps):
        o, s, km = _hip.la_fwd(q, k, v, q_rope, k_rope, scale, eps, _FLAGS)
        ctx.save_for_backward(q, k, q_rope, k_rope, v, s, km)
        ctx.scale = scale
        ctx.eps = eps
        return o

    @staticmethod
    @contiguous
    def backward(ctx, do):
        q, k, q_rope, k_rope, v, s, km = ctx.saved_tensors
        dq, dk, dv, dq_rope, dk_rope = _hip.la_bwd(q, k, v, q_rope, k_rope, do, s, km, ctx.scale,
                                                   ctx.eps, _FLAGS)
        return dq, dk, dq_rope, dk_rope, dv, None, None


def decoupled_la(
    q: torch.Tensor,
    k: torch.Tensor,
    q_rope: torch.Tensor,
    k_rope: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    eps: float = 1e-6
) -> torch.Tensor:
    r"""
    Args:
        q, q_rope: plain (denominator) and rotary (numerator) queries `(B, H, L, K)`
        k, k_rope: plain and rotary keys `(B, H, Lk, K)`; `Lk` may differ from `L` (the reference
            takes one length from q, decoupled.py:413-420)
        v: values `(B, H, Lk, V)`
        scale: defaults to `1 / Lk` (decoupled.py:539-540)
        eps: constant added to the denominator.
    """
    # RoPE modules hand back fp32 features next to 16-bit q, k (layers/mlla.py:32-36 of the
    # reference): they are rounded to the type of q here (the kernels read one element type);
    # the cast is differentiable, so their gradients come back in fp32.
    if isinstance(q, torch.Tensor) and isinstance(q_rope, torch.Tensor) and isinstance(k_rope, torch.Tensor):
        if q_rope.dtype != q.dtype and q_rope.is_floating_point():
            q_rope = q_rope.to(q.dtype)
        if k_rope.dtype != q.dtype and k_rope.is_floating_point():
            k_rope = k_rope.to(q.dtype)
    check_dense("decoupled_la", q, k, v, extra=(q_rope, k_rope))
    if scale is None:
        scale = k.shape[-2] ** -1.0
    return DecoupledLAFunction.apply(q, k, q_rope, k_rope, v, scale, eps)
