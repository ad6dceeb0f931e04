"""BASELINE.json's full sizes on the GPU: parity on sampled heads against the float64
oracle, plus size-independent properties of the operator (constant values, joint
permutation of keys and values, linearity in v, Euler identities of the gradients,
run-to-run determinism, packed == dense)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import TOL, assert_parity, max_rel_err, np64
from oracle import closed_form as cf
from oracle import piecewise as pw

pytestmark = pytest.mark.gpu


def _gpu_inputs(shape_qk, shape_v, dtype, seed=42):
    g = torch.Generator(device="cuda").manual_seed(seed)
    q = (F.elu(torch.randn(shape_qk, generator=g, device="cuda")) + 1).to(dtype)
    k = (F.elu(torch.randn(shape_qk, generator=g, device="cuda")) + 1).to(dtype)
    v = torch.randn(shape_v, generator=g, device="cuda").to(dtype)
    do = torch.randn(shape_v, generator=g, device="cuda").to(dtype)
    return q, k, v, do


@pytest.mark.parametrize("T", [1024, 4096, 16384, 32768])
def test_headline_shape_sampled_heads(T):
    """config 2: B=8, H=16, D=64, fp16, fused forward+backward."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    dtype = torch.float16
    q, k, v, do = _gpu_inputs((8, 16, T, 64), (8, 16, T, 64), dtype)
    leaves = [t.clone().requires_grad_() for t in (q, k, v)]
    o = linear_attention(*leaves, eps=1e-6)
    o.backward(do)
    for b, h in ((0, 0), (3, 7), (7, 15)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = cf.dense_backward(np64(q[sl]), np64(k[sl]), np64(v[sl]), np64(do[sl]), 1.0 / T)
        assert_parity(o[sl], ref["o"], dtype, f"o[{b},{h}]")
        for name, t in zip(("dq", "dk", "dv"), leaves):
            assert_parity(t.grad[sl], ref[name], dtype, f"{name}[{b},{h}]", ref.get(name + "_mag"))


def test_headline_properties():
    from flash_bla.ops.linear_attn.fused import linear_attention
    dtype, T = torch.float16, 16384
    q, k, v, do = _gpu_inputs((8, 16, T, 64), (8, 16, T, 64), dtype)
    o = linear_attention(q, k, v)
    # run-to-run determinism
    assert torch.equal(o, linear_attention(q, k, v))
    # constant values: o = c z / (z + eps), z = q . mean(k)  (exactly representable c)
    c = torch.full_like(v, 1.5)
    z = (q.float() @ k.float().mean(-2, keepdim=True).transpose(-1, -2))
    assert max_rel_err(linear_attention(q, k, c), (1.5 * z / (z + 1e-6)).expand_as(v)) <= TOL[dtype]
    # joint permutation of the (k, v) rows
    perm = torch.randperm(T, device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    o_perm = linear_attention(q, k[:, :, perm].contiguous(), v[:, :, perm].contiguous())
    assert max_rel_err(o_perm, o.float()) <= TOL[dtype]
    # linearity in v (2v and v1 + v2 with exactly representable sums)
    assert max_rel_err(linear_attention(q, k, 2 * v), 2 * o.float()) <= TOL[dtype]
    v2 = torch.roll(v, 1, dims=2)
    lhs = linear_attention(q, k, (v.float() + v2.float()).to(dtype))
    rhs = o.float() + linear_attention(q, k, v2).float()
    assert max_rel_err(lhs, rhs) <= 2 * TOL[dtype]


def test_headline_gradient_identities():
    """With eps = 0 the output is homogeneous of degree 0 in q and in k and linear in v:
    sum(q*dq) = 0, sum(k*dk) = 0 and sum(v*dv) = sum(o*dO), per head."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    q, k, v, do = _gpu_inputs((8, 16, 16384, 64), (8, 16, 16384, 64), torch.float16)
    leaves = [t.clone().requires_grad_() for t in (q, k, v)]
    o = linear_attention(*leaves, eps=0.0)
    o.backward(do)
    dq, dk, dv = (t.grad.double() for t in leaves)
    scale_q = (q.double().abs() * dq.abs()).sum((-1, -2))
    scale_k = (k.double().abs() * dk.abs()).sum((-1, -2))
    assert ((q.double() * dq).sum((-1, -2)).abs() <= 2e-3 * scale_q).all()
    assert ((k.double() * dk).sum((-1, -2)).abs() <= 2e-3 * scale_k).all()
    lhs = (v.double() * dv).sum((-1, -2))
    rhs = (o.double() * do.double()).sum((-1, -2))
    assert ((lhs - rhs).abs() <= 2e-3 * (v.double().abs() * dv.abs()).sum((-1, -2))).all()


@pytest.mark.parametrize("D", [64, 128])
def test_packed_config_full_size(D):
    """config 3: 64 sequences with lengths U[256, 2048], H=16, bf16, forward+backward."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    dtype = torch.bfloat16
    lengths = torch.randint(256, 2049, (64,), generator=torch.Generator().manual_seed(42))
    cu = torch.cat([torch.zeros(1, dtype=torch.int32), torch.cumsum(lengths, 0).to(torch.int32)]).cuda()
    total = int(lengths.sum())
    q, k, v, do = _gpu_inputs((total, 16, D), (total, 16, D), dtype)
    leaves = [t.clone().requires_grad_() for t in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu, int(lengths.max()))
    o.backward(do)
    bounds = cu.tolist()
    for i in (0, 17, 63):
        b, e = bounds[i], bounds[i + 1]
        ref = cf.dense_backward(*(np64(t[b:e, :2].transpose(0, 1)) for t in (q, k, v, do)), 1.0 / (e - b))
        assert_parity(o[b:e, :2].transpose(0, 1), ref["o"], dtype, f"o seq {i}")
        for name, t in zip(("dq", "dk", "dv"), leaves):
            assert_parity(t.grad[b:e, :2].transpose(0, 1), ref[name], dtype, f"{name} seq {i}",
                          ref.get(name + "_mag"))
    # the packed operator on one sequence equals the dense operator on it (bitwise-close)
    b, e = bounds[5], bounds[6]
    dense = linear_attention(*(t[b:e].transpose(0, 1)[None].contiguous() for t in (q, k, v)))
    assert max_rel_err(o[b:e], dense[0].transpose(0, 1).float()) <= 2 ** -7


def test_piecewise_config_full_size():
    """config 5: B=1, H=24, T=16384, D=128, bf16, 64-token blocks, density 0.25 (one head
    against the dense float64 oracle with the same selection)."""
    from flash_bla.ops.piecewise_attn.kernel import (chunk_reduce_fp32, piecewise_sparse_attention,
                                                     select_blocks)
    dtype = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(42)
    q, k, v = (torch.randn(1, 24, 16384, 128, generator=g, device="cuda").to(dtype) for _ in range(3))
    qc, kc, vc, h, _ = chunk_reduce_fp32(q, k, v, 64)
    indices = select_blocks(qc, kc, 128 ** -0.5, 0.25)
    assert indices.shape == (1, 24, 256, 64)
    o = piecewise_sparse_attention(q, k, v, density=0.25, indices=indices)
    assert torch.isfinite(o).all()
    hd = 11
    ref = pw.piecewise_forward(np64(q)[0, hd], np64(k)[0, hd], np64(v)[0, hd], indices[0, hd].cpu().numpy(), 64)
    assert_parity(o[0, hd], ref, dtype, "piecewise head 11")
    rq, rk, rv, _, rH, _ = pw.chunk_reduce(np64(q)[0, hd], np64(k)[0, hd], np64(v)[0, hd], 64)
    assert max_rel_err(h[0, hd], rH) < 1e-4 and max_rel_err(kc[0, hd], rk) < 1e-5


def test_more_than_2_31_elements_per_tensor():
    """B=2, H=16, T=1048576, D=64 fp16: 2^31 elements (4 GiB) per tensor, so every element
    offset of the second batch entry needs more than 31 bits.  Sampled heads from both ends
    against the float64 oracle, forward and backward."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    dtype, B, H, T, D = torch.float16, 2, 16, 1 << 20, 64
    g = torch.Generator(device="cuda").manual_seed(7)
    q = torch.empty(B, H, T, D, dtype=dtype, device="cuda")
    k = torch.empty_like(q)
    v = torch.empty_like(q)
    do = torch.empty_like(q)
    for b in range(B):  # filled per batch entry: the fp32 temporaries stay small
        q[b] = (F.elu(torch.randn(H, T, D, generator=g, device="cuda")) + 1).to(dtype)
        k[b] = (F.elu(torch.randn(H, T, D, generator=g, device="cuda")) + 1).to(dtype)
        v[b] = torch.randn(H, T, D, generator=g, device="cuda").to(dtype)
        do[b] = torch.randn(H, T, D, generator=g, device="cuda").to(dtype)
    assert q.numel() >= 2 ** 31
    leaves = [t.requires_grad_() for t in (q, k, v)]
    o = linear_attention(*leaves)
    o.backward(do)
    torch.cuda.synchronize()
    for b, h in ((0, 0), (1, 0), (1, 15)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = cf.dense_backward(np64(q[sl].detach()), np64(k[sl].detach()), np64(v[sl].detach()), np64(do[sl]),
                                1.0 / T)
        assert_parity(o[sl], ref["o"], dtype, f"o[{b},{h}]")
        for name, t in zip(("dq", "dk", "dv"), leaves):
            assert_parity(t.grad[sl], ref[name], dtype, f"{name}[{b},{h}]", ref.get(name + "_mag"))
