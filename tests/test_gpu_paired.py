"""Two queries on shared keys and values (paired_linear_attention, fbla_la_pair_fwd/bwd) against the
float64 oracle: by definition the pair of independent operator calls of
flash_bla/layers/polaformer.py:89-90, whose key and value gradients add up."""
import numpy as np
import pytest
import torch

from helpers import assert_parity, make_qkv, np64
from oracle import closed_form as cf

pytestmark = pytest.mark.gpu


def _oracle(q1, q2, k, v, do1, do2, scale, eps=1e-6):
    half = v.shape[-1] // 2
    r1 = cf.dense_backward(np64(q1), np64(k), np64(v[..., :half]), np64(do1), scale, eps)
    r2 = cf.dense_backward(np64(q2), np64(k), np64(v[..., half:]), np64(do2), scale, eps)
    return dict(o1=r1["o"], o2=r2["o"], dq1=r1["dq"], dq2=r2["dq"], dk=r1["dk"] + r2["dk"],
                dv=np.concatenate([r1["dv"], r2["dv"]], -1),
                dq1_mag=r1["dq_mag"], dq2_mag=r2["dq_mag"], dk_mag=np.maximum(r1["dk_mag"], r2["dk_mag"]))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("B,H,L,DK,DV", [(2, 3, 300, 128, 64), (1, 2, 5000, 128, 64), (2, 2, 777, 64, 64),
                                         (1, 4, 1030, 32, 32), (1, 2, 64, 128, 128), (1, 1, 9000, 64, 128),
                                         (1, 2, 200, 96, 48)])
def test_paired_matches_two_independent_calls(dtype, B, H, L, DK, DV):
    from flash_bla import _hip
    from flash_bla.ops.linear_attn.paired import paired_linear_attention
    q1, k, v, do, q2 = make_qkv((B, H, L, DK), (B, H, L, DV), dtype, seed=L + DK, n_extra=1)
    half = DV // 2
    do1, do2 = do[..., :half].contiguous(), do[..., half:].contiguous()
    leaves = [t.cuda().requires_grad_() for t in (q1, q2, k, v)]
    assert _hip.pair_supported(leaves[0], leaves[3])
    o1, o2 = paired_linear_attention(*leaves)
    torch.autograd.backward([o1, o2], [do1.cuda(), do2.cuda()])
    ref = _oracle(q1, q2, k, v, do1, do2, 1.0 / L)
    assert_parity(o1, ref["o1"], dtype, "o1")
    assert_parity(o2, ref["o2"], dtype, "o2")
    for name, leaf in zip(("dq1", "dq2", "dk", "dv"), leaves):
        assert_parity(leaf.grad, ref[name], dtype, name, ref.get(name + "_mag"))


def test_paired_explicit_scale_and_eps():
    from flash_bla.ops.linear_attn.paired import paired_linear_attention
    dtype = torch.float16
    q1, k, v, do, q2 = make_qkv((1, 2, 400, 128), (1, 2, 400, 64), dtype, seed=3, n_extra=1)
    leaves = [t.cuda().requires_grad_() for t in (q1, q2, k, v)]
    o1, o2 = paired_linear_attention(*leaves, scale=0.01, eps=1e-3)
    do1, do2 = do[..., :32].contiguous(), do[..., 32:].contiguous()
    torch.autograd.backward([o1, o2], [do1.cuda(), do2.cuda()])
    ref = _oracle(q1, q2, k, v, do1, do2, 0.01, 1e-3)
    assert_parity(o1, ref["o1"], dtype, "o1")
    assert_parity(o2, ref["o2"], dtype, "o2")
    for name, leaf in zip(("dq1", "dq2", "dk", "dv"), leaves):
        assert_parity(leaf.grad, ref[name], dtype, name, ref.get(name + "_mag"))


@pytest.mark.parametrize("case", ["fp32", "fewer_keys", "odd_half"])
def test_paired_shapes_outside_the_shared_kernels_run_the_two_calls(case):
    """fp32 and another number of keys than queries run the two operator calls, halves that are not
    multiples of 8 zero-padded copies on the shared kernels: same results."""
    from flash_bla import _hip
    from flash_bla.ops.linear_attn.paired import paired_linear_attention
    dtype = torch.float32 if case == "fp32" else torch.float16
    Lq, Lk = (300, 75) if case == "fewer_keys" else (300, 300)
    DV = 24 if case == "odd_half" else 32
    g = torch.Generator().manual_seed(11)
    feat = lambda *s: (torch.nn.functional.elu(torch.randn(*s, generator=g)) + 1).to(dtype)  # noqa: E731
    q1, q2, k = feat(1, 2, Lq, 64), feat(1, 2, Lq, 64), feat(1, 2, Lk, 64)
    v = torch.randn(1, 2, Lk, DV, generator=g).to(dtype)
    if case != "fewer_keys":
        assert not _hip.pair_supported(q1.cuda(), v.cuda())
    o1, o2 = paired_linear_attention(q1.cuda(), q2.cuda(), k.cuda(), v.cuda())
    half = DV // 2
    for o, q, vv in ((o1, q1, v[..., :half]), (o2, q2, v[..., half:])):
        ref = cf.dense_forward(np64(q), np64(k), np64(vv), 1.0 / Lk)[0]
        assert_parity(o, ref, dtype, case)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("B,H,L,DK,DV", [(1, 2, 1500, 100, 128), (3, 4, 15, 100, 26), (1, 1, 400, 17, 10)])
def test_paired_head_dims_that_are_not_multiples_of_eight(dtype, B, H, L, DK, DV):
    """Zero-padded copies keep the shared pass over k and v (one rounding of dk instead of the sum of two
    rounded gradients): outputs and all four gradients against the oracle."""
    from flash_bla.ops.linear_attn.paired import paired_linear_attention
    q1, k, v, do, q2 = make_qkv((B, H, L, DK), (B, H, L, DV), dtype, seed=L + DK, n_extra=1)
    half = DV // 2
    do1, do2 = do[..., :half].contiguous(), do[..., half:].contiguous()
    leaves = [t.cuda().requires_grad_() for t in (q1, q2, k, v)]
    o1, o2 = paired_linear_attention(*leaves)
    assert o1.shape == (B, H, L, half) and o2.shape == (B, H, L, half)
    torch.autograd.backward([o1, o2], [do1.cuda(), do2.cuda()])
    ref = _oracle(q1, q2, k, v, do1, do2, 1.0 / L)
    assert_parity(o1, ref["o1"], dtype, "o1")
    assert_parity(o2, ref["o2"], dtype, "o2")
    for name, leaf in zip(("dq1", "dq2", "dk", "dv"), leaves):
        assert leaf.grad.shape == leaf.shape
        assert_parity(leaf.grad, ref[name], dtype, name, ref.get(name + "_mag"))


def test_paired_rejects_mismatched_queries():
    from flash_bla.ops.linear_attn.paired import paired_linear_attention
    x = torch.ones(1, 1, 16, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        paired_linear_attention(x, x[:, :, :8], x, x)
    with pytest.raises(ValueError):
        paired_linear_attention(x, x, x, x[..., :33])
