"""The blocks' feature map elu(x) + 1 as one HIP launch (queries and keys together).

The reference's layers write `F.elu(x) + 1.0` per tensor (layers/linfusion.py:88-89,
layers/mlla.py:74-75): two elementwise torch kernels each.  The same rounding steps as that expression (the bits agree up to
the last place of the two exp routines); the layers' `mode='torch'` keeps the torch expression.
"""
import torch

from flash_bla import _hip


class EluPlusOneFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x0, x1):
        x0 = x0.contiguous()
        x1 = x1.contiguous() if x1 is not None else None
        ctx.save_for_backward(x0, x1)
        if x1 is None:
            return _hip.elu1_fwd(x0), None
        return _hip.elu1_fwd(x0, x1)

    @staticmethod
    def backward(ctx, g0, g1):
        x0, x1 = ctx.saved_tensors
        d0 = _hip.elu1_bwd(x0, g0.contiguous()) if g0 is not None else None
        d1 = _hip.elu1_bwd(x1, g1.contiguous()) if (x1 is not None and g1 is not None) else None
        return d0, d1


def elu_plus_one(x, y=None):
    """elu(x) + 1 (and elu(y) + 1: then a pair is returned) on the GPU.  Floating-point GPU tensors
    of one dtype; non-contiguous inputs are copied first."""
    for t in (x, y):
        if t is not None and not torch.is_tensor(t):
            raise TypeError("elu_plus_one expects tensors")
    if y is not None and (y.dtype != x.dtype or y.device != x.device):
        raise ValueError("elu_plus_one: both tensors must have the same dtype and device")
    if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError(f"elu_plus_one: unsupported dtype {x.dtype}")
    out = EluPlusOneFunction.apply(x, y)
    return out[0] if y is None else out
