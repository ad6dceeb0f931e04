"""Two queries on shared keys and values: the pair of operator calls at the heart of PolaFormer
(flash_bla/layers/polaformer.py:89-90)

    x_sim = linear_attention(q_sim, k, v1)        x_opp = linear_attention(q_opp, k, v2)

with `v1 | v2` the two halves of the value channels, as one autograd node: the state
`S = scale * K^T [v1 | v2]` and `km` come from one pass over k and v, each query multiplies its
half of the state's columns, and the backward reads k and v once and writes `dk` (the sum of the
two calls' key gradients) once.  Not in the reference, which runs the two calls independently.
"""
from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from flash_bla import _hip
from flash_bla.ops._check import check_dense
from flash_bla.ops.linear_attn.fused import linear_attention
from flash_bla.utils import contiguous


class PairedLinearAttnFunction(torch.autograd.Function):
    @staticmethod
    @contiguous
    def forward(ctx, q1, q2, k, v, scale, eps):
        o1, o2, s, km = _hip.pair_fwd(q1, q2, k, v, scale, eps)
        ctx.save_for_backward(q1, q2, k, v, s, km)
        ctx.scale = scale
        ctx.eps = eps
        return o1, o2

    @staticmethod
    @contiguous
    def backward(ctx, do1, do2):
        q1, q2, k, v, s, km = ctx.saved_tensors
        dq1, dq2, dk, dv = _hip.pair_bwd(q1, q2, k, v, do1, do2, s, km, ctx.scale, ctx.eps)
        return dq1, dq2, dk, dv, None, None


def paired_linear_attention(
    q1: torch.Tensor,
    q2: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    eps: float = 1e-6,
) -> Tuple[torch.Tensor, torch.Tensor]:
    r"""
    Args:
        q1, q2: two sets of queries `(B, H, L, K)`
        k: keys `(B, H, L, K)` shared by both
        v: values `(B, H, L, V)` with V even: `q1` attends to `v[..., :V/2]`, `q2` to `v[..., V/2:]`
        scale: factor on the key-value state, default `1 / L`; eps: added to the denominators.
    Returns `(o1, o2)`, each `(B, H, L, V/2)`:
    `linear_attention(q1, k, v[..., :V/2])` and `linear_attention(q2, k, v[..., V/2:])`.
    fp16 / bf16 with as many keys as queries take the shared-state kernels (K and V/2 that are not
    multiples of 8 through zero-padded copies); everything else runs the two operator calls.
    """
    check_dense("paired_linear_attention", q1, k, v)
    if q2.shape != q1.shape or q2.dtype != q1.dtype or q2.device != q1.device:
        raise ValueError("paired_linear_attention: q1 and q2 must agree in shape, dtype and device")
    if v.shape[-1] % 2:
        raise ValueError("paired_linear_attention: the value dim must be even")
    if scale is None:
        scale = k.shape[-2] ** -1.0
    v1, v2 = v.chunk(2, dim=-1)
    if k.shape[-2] == q1.shape[-2]:
        if _hip.pair_supported(q1, v):
            return PairedLinearAttnFunction.apply(q1, q2, k, v, scale, eps)
        # head dims that are not multiples of 8: zero features up to the next multiple change nothing
        # (zero key features add nothing to any product, zero value columns give zero output columns)
        # and keep the one pass over k and v, with its single rounding of dk
        half = v.shape[-1] // 2
        kw, hw = -(-q1.shape[-1] // 8) * 8, -(-half // 8) * 8
        if q1.dtype != torch.float32 and (kw, hw) != (q1.shape[-1], half):
            widen = lambda t, n: F.pad(t, (0, n - t.shape[-1]))
            vw = torch.cat([widen(v1, hw), widen(v2, hw)], dim=-1)
            q1w, q2w, kwide = (widen(t, kw) for t in (q1, q2, k))
            if _hip.pair_supported(q1w, vw):
                o1, o2 = PairedLinearAttnFunction.apply(q1w, q2w, kwide, vw, scale, eps)
                return o1[..., :half], o2[..., :half]
    return linear_attention(q1, k, v1.contiguous(), scale, eps), linear_attention(q2, k, v2.contiguous(), scale, eps)
