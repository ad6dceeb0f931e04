"""Seeded input generation and error metrics shared by the tests."""
import numpy as np
import torch
import torch.nn.functional as F


def make_qkv(shape_qk, shape_v, dtype=torch.float32, seed=42, n_extra=0):
    """q,k = elu(N(0,1))+1, v,dO ~ N(0,1): drawn on the CPU in fp32 from a seeded
    generator, then rounded to `dtype` (the distribution of
    tests/ops/test_varlen_linear_attn.py:25-28)."""
    g = torch.Generator().manual_seed(seed)
    q = (F.elu(torch.randn(shape_qk, generator=g)) + 1).to(dtype)
    k = (F.elu(torch.randn(shape_qk, generator=g)) + 1).to(dtype)
    v = torch.randn(shape_v, generator=g).to(dtype)
    do = torch.randn(shape_v, generator=g).to(dtype)
    extra = [(F.elu(torch.randn(shape_qk, generator=g)) + 1).to(dtype) for _ in range(n_extra)]
    return (q, k, v, do, *extra)


def max_rel_err(x, ref):
    """max|x - ref| / max|ref| on float64 copies."""
    x = np.asarray(x.detach().double().cpu() if isinstance(x, torch.Tensor) else x, dtype=np.float64)
    ref = np.asarray(ref.detach().double().cpu() if isinstance(ref, torch.Tensor) else ref, dtype=np.float64)
    denom = max(np.abs(ref).max(), 1e-30)
    return float(np.abs(x - ref).max() / denom)


def np64(t):
    return t.detach().double().cpu().numpy()


# Parity gates (max|x-ref|/max|ref| against the float64 oracle evaluated on the
# same, already-rounded inputs): fp32 accumulation of 16-bit inputs <= 2e-3,
# fp32 inputs <= 1e-5.
TOL = {torch.float16: 2e-3, torch.bfloat16: 2e-3, torch.float32: 1e-5}
