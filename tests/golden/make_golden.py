"""Writes tests/golden/*.npz: small seeded inputs with float64 outputs and gradients.

The reference repository ships no golden vectors for these operators; these
fixtures are produced by the pinned CPU oracle (oracle/closed_form.py, itself
checked against brute force, autograd and invariants in tests/test_oracle.py).
Inputs are rounded to fp16 first so that the same bits can be fed to fp16, bf16
(after a second rounding, done by the test) and fp32 kernels.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from helpers import make_qkv, np64  # noqa: E402
from oracle import closed_form as cf  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def _slim(name, a):
    """Term magnitudes are only used through their maximum: keep one value per token."""
    return a.max(axis=-1, keepdims=True) if name.endswith("_mag") else a


def dense_case(name, B, H, L, DK, DV, scale, eps, normalize, decoupled, seed):
    q, k, v, do, qr, kr = make_qkv((B, H, L, DK), (B, H, L, DV), torch.float16, seed, n_extra=2)
    arrs = {n: np64(t).astype(np.float32) for n, t in dict(q=q, k=k, v=v, do=do).items()}
    kw = {}
    if decoupled:
        arrs["q_rope"], arrs["k_rope"] = np64(qr).astype(np.float32), np64(kr).astype(np.float32)
        kw = dict(q_rope=arrs["q_rope"], k_rope=arrs["k_rope"])
    s = (1.0 / L if normalize else DK ** -0.5) if scale is None else scale
    g = cf.dense_backward(arrs["q"], arrs["k"], arrs["v"], arrs["do"], s, eps, normalize, **kw)
    out = dict(arrs)
    out.update({"ref_" + n: _slim(n, a) for n, a in g.items()})
    out["meta"] = np.array([s, eps, float(normalize), float(decoupled)])
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)


def varlen_case(name, lengths, H, DK, DV, scale, eps, seed):
    T = int(sum(lengths))
    q, k, v, do = make_qkv((T, H, DK), (T, H, DV), torch.float16, seed)
    arrs = {n: np64(t).astype(np.float32) for n, t in dict(q=q, k=k, v=v, do=do).items()}
    cu = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    g = cf.varlen_backward(arrs["q"], arrs["k"], arrs["v"], arrs["do"], cu, scale, eps)
    out = dict(arrs)
    out.update({"ref_" + n: _slim(n, a) for n, a in g.items()})
    out["cu_seqlens"] = cu
    out["meta"] = np.array([-1.0 if scale is None else scale, eps])
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)


if __name__ == "__main__":
    dense_case("linear_attn_b1h2l37_dk16_dv8", 1, 2, 37, 16, 8, None, 1e-6, True, False, 101)
    dense_case("linear_attn_b1h2l70_dk64_dv64", 1, 2, 70, 64, 64, None, 1e-6, True, False, 102)
    dense_case("simple_la_b1h2l50_dk32_dv16", 1, 2, 50, 32, 16, None, 0.0, False, False, 103)
    dense_case("decoupled_b1h2l45_dk32_dv32", 1, 2, 45, 32, 32, None, 1e-6, True, True, 104)
    varlen_case("varlen_8_17_32_h2_dk17_dv13", [8, 17, 32], 2, 17, 13, None, 1e-6, 105)
    varlen_case("varlen_5_64_1_h3_dk64_dv48", [5, 64, 1], 3, 64, 48, 0.02, 1e-6, 106)
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
