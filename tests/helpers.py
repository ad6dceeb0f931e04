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


def _scale_of(ref, floor):
    return max(float(np.abs(ref).max()), 0.0 if floor is None else float(np.abs(floor).max()), 1e-30)


def max_rel_err(x, ref, floor=None):
    """max|x - ref| / max|ref| on float64 copies (`floor`: see parity_errors)."""
    x = np.asarray(x.detach().double().cpu() if isinstance(x, torch.Tensor) else x, dtype=np.float64)
    ref = np.asarray(ref.detach().double().cpu() if isinstance(ref, torch.Tensor) else ref, dtype=np.float64)
    return float(np.abs(x - ref).max() / _scale_of(ref, floor))


def np64(t):
    return t.detach().double().cpu().numpy()


# Parity gates, all on float64 copies against the float64 oracle evaluated on the
# same, already-rounded inputs.
#
#   plain  = max|x - ref| / max|ref|
#   excess = max(|x - ref| - u*|ref|, 0) / max|ref|     u = unit roundoff of the OUTPUT dtype
#
# `excess` removes the unavoidable rounding of the result to its storage type
# (u = 2^-11 for fp16, 2^-8 for bf16): it measures the arithmetic itself, i.e. the
# "fp32 accumulation of 16-bit inputs" error, and is gated at 2e-3 like `plain`.
# For bf16 a correctly rounded result already reaches plain = 2^-8 = 3.9e-3, so
# its plain gate is 2e-3 + 2^-8; fp16 and fp32 use 2e-3 and 1e-5 directly.
UNIT_ROUNDOFF = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8, torch.float32: 2.0 ** -24}
TOL = {torch.float16: 2e-3, torch.bfloat16: 2e-3 + 2.0 ** -8, torch.float32: 1e-5}
TOL_EXCESS = {torch.float16: 2e-3, torch.bfloat16: 2e-3, torch.float32: 1e-5}


def excess_err(x, ref, dtype, floor=None):
    x = np.asarray(x.detach().double().cpu() if isinstance(x, torch.Tensor) else x, dtype=np.float64)
    ref = np.asarray(ref.detach().double().cpu() if isinstance(ref, torch.Tensor) else ref, dtype=np.float64)
    denom = _scale_of(ref, floor)
    return float(np.maximum(np.abs(x - ref) - UNIT_ROUNDOFF[dtype] * np.abs(ref), 0.0).max() / denom)


def parity_errors(x, ref, dtype, floor=None):
    """(plain, excess, ok) for one tensor.  `floor` (the oracle's dq_mag / dk_mag)
    widens the scale max|ref| to the size of the terms that were added to form
    ref, for gradients that cancel (sequences of one or two tokens)."""
    plain, excess = max_rel_err(x, ref, floor), excess_err(x, ref, dtype, floor)
    ok = plain <= TOL[dtype] and excess <= TOL_EXCESS[dtype]
    return plain, excess, ok


def assert_parity(x, ref, dtype, what="", floor=None):
    plain, excess, ok = parity_errors(x, ref, dtype, floor)
    assert ok, (f"{what}: plain {plain:.3e} (gate {TOL[dtype]:.3e}), "
                f"excess {excess:.3e} (gate {TOL_EXCESS[dtype]:.3e})")
    return plain, excess
