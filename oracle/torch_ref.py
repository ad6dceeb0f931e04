"""Torch restatement of the reference's naive (torch) operators.

Test infrastructure only (see oracle/__init__.py).  Each function follows the
cited reference lines; inputs may live on any device and have any float dtype.
"""
import torch


def naive_linear_attn(q, k, v, scale=None, eps=1e-6):
    """flash_bla/ops/linear_attn/naive.py:6-14 (eps is hard-coded to 1e-6 there)."""
    if scale is None:
        scale = k.shape[-2] ** -1.0
    z = q @ k.mean(dim=-2, keepdim=True).transpose(-2, -1)
    s = k.transpose(-2, -1) @ (v * scale)
    return q @ s / (z + eps)


def naive_decoupled_la(q, k, q_rope, k_rope, v, scale=None, eps=1e-6):
    """flash_bla/ops/linear_attn/naive.py:17-25."""
    if scale is None:
        scale = k.shape[-2] ** -1.0
    z = q @ k.mean(dim=-2, keepdim=True).transpose(-2, -1)
    s = k_rope.transpose(-2, -1) @ (v * scale)
    return q_rope @ s / (z + eps)


def naive_varlen_linear_attn(q, k, v, cu_seqlens, scale=None, eps=1e-6):
    """flash_bla/ops/linear_attn/naive.py:28-43 (packed [T,H,D] layout)."""
    bounds = [int(x) for x in cu_seqlens.tolist()]
    outs = []
    for bos, eos in zip(bounds[:-1], bounds[1:]):
        n = eos - bos
        s_i = n ** -1.0 if scale is None else scale
        qi = q[bos:eos].transpose(0, 1)
        ki = k[bos:eos].transpose(0, 1)
        vi = v[bos:eos].transpose(0, 1)
        z = (qi * ki.mean(dim=1)[:, None, :]).sum(dim=-1, keepdim=True)
        s = ki.transpose(-2, -1) @ (vi * s_i)
        outs.append(((qi @ s) / (z + eps)).transpose(0, 1))
    return torch.cat(outs, dim=0)


def naive_simple_la(q, k, v, scale=None):
    """flash_bla/ops/simple_la/naive.py:8-20."""
    if scale is None:
        scale = q.shape[-1] ** -0.5
    s = k.transpose(-2, -1) @ (v * scale)
    return q @ s


def linfusion_torch_mode(q, k, v, eps=1e-4):
    """flash_bla/layers/linfusion.py:92-96 (the layer's own torch formula)."""
    L = k.shape[-2]
    z = q @ k.mean(dim=-2, keepdim=True).transpose(-2, -1) + eps
    kv = (k.transpose(-2, -1) * (L ** -0.5)) @ (v * (L ** -0.5))
    return q @ kv / z
