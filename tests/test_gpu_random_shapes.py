"""Seeded random shapes through every operator family and dtype against the float64 oracle:
head dims drawn from the sets the kernels specialise on and from outside them, lengths from
one token to a few chunks, packed batches with empty and one-token sequences."""
import numpy as np
import pytest
import torch

from helpers import assert_parity, make_qkv, np64, parity_errors
from oracle import closed_form as cf

pytestmark = pytest.mark.gpu

DIMS = [64, 64, 64, 128, 32, 16, 8, 24, 100]
DTYPES = [torch.float16, torch.bfloat16, torch.float32]


def _dense_case(rng):
    variant = rng.choice(["linear", "simple", "decoupled"], p=[0.5, 0.3, 0.2])
    DK, DV = int(rng.choice(DIMS)), int(rng.choice(DIMS))
    if rng.random() < 0.5:
        DV = DK
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 6))
    L = int(rng.choice([1, 2, 7, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 255, 257, 500, 1000, 2049, 5000]))
    dtype = DTYPES[int(rng.integers(0, 3))]
    return variant, B, H, L, DK, DV, dtype


@pytest.mark.parametrize("seed", range(6))
def test_random_dense_cases(seed):
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.simple_la.fused import simple_la
    rng = np.random.default_rng(1000 + seed)
    for case in range(12):
        variant, B, H, L, DK, DV, dtype = _dense_case(rng)
        q, k, v, do, qr, kr = make_qkv((B, H, L, DK), (B, H, L, DV), dtype, seed * 100 + case, n_extra=2)
        normalize = variant != "simple"
        scale = 1.0 / L if normalize else DK ** -0.5
        kw = dict(q_rope=np64(qr), k_rope=np64(kr)) if variant == "decoupled" else {}
        ref = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), scale, 1e-6, normalize, **kw)
        tensors = (q, k, qr, kr, v) if variant == "decoupled" else (q, k, v)
        leaves = [t.cuda().requires_grad_() for t in tensors]
        if variant == "linear":
            o = linear_attention(*leaves)
            names = ["dq", "dk", "dv"]
        elif variant == "simple":
            o = simple_la(*leaves)
            names = ["dq", "dk", "dv"]
        else:
            o = decoupled_la(*leaves)
            names = ["dq", "dk", "dq_rope", "dk_rope", "dv"]
        o.backward(do.cuda())
        tag = f"{variant} {dtype} B{B} H{H} L{L} DK{DK} DV{DV}"
        errs = {"o": parity_errors(o, ref["o"], dtype)}
        for name, t in zip(names, leaves):
            errs[name] = parity_errors(t.grad, ref[name], dtype, ref.get(name + "_mag"))
        bad = {n: e for n, e in errs.items() if not e[2]}
        assert not bad, f"{tag}: {errs}"


@pytest.mark.parametrize("seed", range(4))
def test_random_packed_cases(seed):
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    rng = np.random.default_rng(2000 + seed)
    for case in range(8):
        D = int(rng.choice([64, 64, 128, 32, 48]))
        H = int(rng.integers(1, 9))
        nseq = int(rng.integers(1, 12))
        lengths = [int(rng.choice([0, 1, 1, 3, 15, 16, 17, 40, 64, 129, 300, 777, 1500])) for _ in range(nseq)]
        if sum(lengths) == 0:
            lengths[0] = 5
        dtype = DTYPES[int(rng.integers(0, 3))]
        T = sum(lengths)
        q, k, v, do = make_qkv((T, H, D), (T, H, D), dtype, seed * 100 + case)
        cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32).cuda()
        leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
        o = varlen_linear_attention(*leaves, cu, max(lengths))
        o.backward(do.cuda())
        ref = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.cpu().numpy())
        tag = f"{dtype} H{H} D{D} lengths{lengths}"
        assert_parity(o, ref["o"], dtype, f"o {tag}")
        for name, t in zip(("dq", "dk", "dv"), leaves):
            for b, e in zip(cu[:-1].tolist(), cu[1:].tolist()):
                if e > b:
                    floor = ref[name + "_mag"][b:e] if name + "_mag" in ref else None
                    assert_parity(t.grad[b:e], ref[name][b:e], dtype, f"{name}[{b}:{e}] {tag}", floor)
