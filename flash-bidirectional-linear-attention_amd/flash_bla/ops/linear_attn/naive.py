"""Plain-torch formulas of the operators (counterpart of
flash_bla/ops/linear_attn/naive.py).  They run on whatever device their inputs
live on and are what the layers' ``mode='torch'`` uses; the HIP operators never
call them."""
import torch


def naive_linear_attn(q, k, v, scale=None):
    if scale is None:
        scale = k.shape[-2] ** -1.0
    z = q @ k.mean(dim=-2, keepdim=True).transpose(-2, -1)
    s = k.transpose(-2, -1) @ (v * scale)
    return q @ s / (z + 1e-6)


def naive_decoupled_la(q, k, q_rope, k_rope, v, scale=None):
    if scale is None:
        scale = k.shape[-2] ** -1.0
    z = q @ k.mean(dim=-2, keepdim=True).transpose(-2, -1)
    s = k_rope.transpose(-2, -1) @ (v * scale)
    return q_rope @ s / (z + 1e-6)


def naive_varlen_linear_attn(q, k, v, cu_seqlens, scale=None, eps=1e-6):
    bounds = cu_seqlens.tolist()
    outputs = []
    for bos, eos in zip(bounds[:-1], bounds[1:]):
        seq_scale = (eos - bos) ** -1.0 if scale is None else scale
        q_i, k_i, v_i = (x[bos:eos].transpose(0, 1) for x in (q, k, v))
        z = (q_i * k_i.mean(dim=1)[:, None, :]).sum(dim=-1, keepdim=True)
        s = k_i.transpose(-2, -1) @ (v_i * seq_scale)
        outputs.append(((q_i @ s) / (z + eps)).transpose(0, 1))
    return torch.cat(outputs, dim=0)
