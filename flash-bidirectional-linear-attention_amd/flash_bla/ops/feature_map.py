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


ELU_PLUS_ONE = "elu+1"


def check_feature_map(feature_map):
    """The operators' `feature_map` argument: None or "elu+1"."""
    if feature_map is not None and feature_map != ELU_PLUS_ONE:
        raise ValueError(f'feature_map must be None or "{ELU_PLUS_ONE}", got {feature_map!r}')
    return feature_map is not None


def mapped_in_kernels(q, v):
    """16-bit heads of 64 x 64: the shapes for which the attention kernels take part in the feature
    map (on load in an inference forward, on the gradients in a backward)."""
    return q.dtype in (torch.float16, torch.bfloat16) and q.shape[-1] == 64 and v.shape[-1] == 64


def applied_on_load(q, k, v):
    """True when a plain forward call suffices: the kernels apply elu(x) + 1 to q and k as they
    load them (16-bit heads of 64 x 64) and nothing is to be differentiated (a call that records a
    graph goes through the autograd nodes, whose backward kernels map on load as well)."""
    if not mapped_in_kernels(q, v):
        return False
    return not (torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v)))
