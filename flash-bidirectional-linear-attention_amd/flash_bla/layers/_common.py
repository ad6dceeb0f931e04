"""Pieces shared by the layer modules."""
import torch

FAST_MODES = ("triton", "hip")  # 'triton' is the reference's name for "the fused operator"


def split_heads(x, heads):
    """(B, N, heads*d) -> contiguous (B, heads, N, d)."""
    b, n, c = x.shape
    return x.view(b, n, heads, c // heads).transpose(1, 2).contiguous()


def merge_heads(x):
    """(B, heads, N, d) -> (B, N, heads*d)."""
    b, h, n, d = x.shape
    return x.transpose(1, 2).reshape(b, n, h * d)


def torch_linear_attention(q, k, v, eps=1e-6, q_num=None, k_num=None):
    """The layers' `mode='torch'` formula: state from the (rotary) numerator features with
    the 1/n split as n^-1/2 on each factor, denominator from the plain features."""
    n = k.shape[-2]
    q_num = q if q_num is None else q_num
    k_num = k if k_num is None else k_num
    z = q @ k.mean(dim=-2, keepdim=True).transpose(-2, -1) + eps
    kv = (k_num.transpose(-2, -1) * n ** -0.5) @ (v * n ** -0.5)
    return (q_num @ kv) / z


def check_mode(mode):
    if mode != "torch" and mode not in FAST_MODES:
        raise NotImplementedError(f"unknown mode {mode!r}")
    return mode != "torch"
