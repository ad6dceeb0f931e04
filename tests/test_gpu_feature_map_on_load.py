"""The operators' `feature_map="elu+1"` argument: q and k are given before the blocks' feature map
(layers/linfusion.py:88-89) and an inference forward of 16-bit heads of 64 x 64 applies it inside
the kernels as they load them.  Checked against the float64 oracle evaluated on the mapped tensors
(mapped the way the reference's layers map them: `F.elu(x) + 1.0` in the tensor's type), against
the path that maps first, through autograd (which must map first), on shapes the kernels do not
cover (which must map first too), and at the C ABI's edges."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import assert_parity, max_rel_err, np64
from oracle import closed_form as cf

pytestmark = pytest.mark.gpu


def _raw(shape_qk, shape_v, dtype, seed, spread=1.5):
    g = torch.Generator().manual_seed(seed)
    q = (spread * torch.randn(shape_qk, generator=g)).to(dtype)
    k = (spread * torch.randn(shape_qk, generator=g)).to(dtype)
    v = torch.randn(shape_v, generator=g).to(dtype)
    return q, k, v


def _mapped(x):
    """The reference layers' expression on a tensor of the inputs' type (computed on the GPU, where
    torch rounds the elu to the type and then the sum)."""
    return (F.elu(x.cuda()) + 1.0).cpu()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("B,H,L", [(2, 3, 300), (1, 2, 1000), (1, 5, 10), (2, 2, 17), (1, 1, 64), (1, 16, 4099),
                                   (8, 16, 2048)])
def test_dense_forward_maps_on_load(B, H, L, dtype):
    from flash_bla.ops.feature_map import elu_plus_one
    from flash_bla.ops.linear_attn.fused import linear_attention
    q, k, v = _raw((B, H, L, 64), (B, H, L, 64), dtype, seed=L)
    with torch.no_grad():
        o = linear_attention(q.cuda(), k.cuda(), v.cuda(), feature_map="elu+1")
        o_two_steps = linear_attention(*elu_plus_one(q.cuda(), k.cuda()), v.cuda())
    assert o.dtype == dtype and o.shape == v.shape
    ref = cf.dense_forward(np64(_mapped(q)), np64(_mapped(k)), np64(v), 1.0 / L)[0]
    assert_parity(o, ref, dtype, f"mapped on load B{B} H{H} L{L}")
    # the two paths differ only in the last place of their exp routines
    assert max_rel_err(o, np64(o_two_steps)) < 2e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("lq,lk", [(300, 75), (64, 1000)])
def test_fewer_or_more_keys_than_queries(lq, lk, dtype):
    from flash_bla.ops.linear_attn.fused import linear_attention
    q, _, _ = _raw((2, 3, lq, 64), (2, 3, lq, 64), dtype, seed=lq)
    _, k, v = _raw((2, 3, lk, 64), (2, 3, lk, 64), dtype, seed=lk)
    with torch.no_grad():
        o = linear_attention(q.cuda(), k.cuda(), v.cuda(), feature_map="elu+1")
    ref = cf.dense_forward(np64(_mapped(q)), np64(_mapped(k)), np64(v), 1.0 / lk)[0]
    assert_parity(o, ref, dtype, f"Lq{lq} Lk{lk}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("lq,lk", [(300, 75), (64, 1000)])
def test_gradients_with_fewer_or_more_keys_than_queries(lq, lk, dtype):
    from flash_bla.ops.linear_attn.fused import linear_attention
    q, _, _ = _raw((2, 3, lq, 64), (2, 3, lq, 64), dtype, seed=lq + 3)
    _, k, v = _raw((2, 3, lk, 64), (2, 3, lk, 64), dtype, seed=lk + 3)
    do = torch.randn(2, 3, lq, 64, generator=torch.Generator().manual_seed(lq)).to(dtype)
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = linear_attention(*leaves, feature_map="elu+1")
    o.backward(do.cuda())
    ref = cf.dense_backward(np64(_mapped(q)), np64(_mapped(k)), np64(v), np64(do), 1.0 / lk)
    dphi = lambda x: np.where(np64(x) > 0, 1.0, np.exp(np.minimum(np64(x), 0.0)))
    assert_parity(o, ref["o"], dtype, "o")
    assert_parity(leaves[0].grad, ref["dq"] * dphi(q), dtype, "dq", ref.get("dq_mag"))
    assert_parity(leaves[1].grad, ref["dk"] * dphi(k), dtype, "dk", ref.get("dk_mag"))
    assert_parity(leaves[2].grad, ref["dv"], dtype, "dv", ref.get("dv_mag"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_unnormalised_forward_maps_on_load(dtype):
    """The C ABI's flag without FBLA_NORMALIZE (the simple_la family)."""
    from flash_bla import _hip
    B, H, L = 2, 3, 777
    q, k, v = _raw((B, H, L, 64), (B, H, L, 64), dtype, seed=5)
    scale = 64 ** -0.5
    o = _hip.la_fwd(q.cuda(), k.cuda(), v.cuda(), None, None, scale, 1e-6, _hip.ELU1_QK)[0]
    ref = cf.dense_forward(np64(_mapped(q)), np64(_mapped(k)), np64(v), scale, normalize=False)[0]
    assert_parity(o, ref, dtype, "simple_la mapped on load")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_packed_forward_maps_on_load(dtype):
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    lens = [5, 300, 1, 64, 1000, 17, 16, 2049]
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    T, H = int(cu[-1]), 4
    q, k, v = _raw((T, H, 64), (T, H, 64), dtype, seed=9)
    with torch.no_grad():
        o = varlen_linear_attention(q.cuda(), k.cuda(), v.cuda(), cu.cuda(), max(lens), feature_map="elu+1")
    ref = cf.varlen_forward(np64(_mapped(q)), np64(_mapped(k)), np64(v), cu.numpy())
    assert_parity(o, ref, dtype, "packed, mapped on load")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_gradients_flow_through_the_feature_map(dtype):
    """With something to differentiate the operator maps q and k first (one launch) and autograd sees
    the map: the gradients are those of the composed function."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    B, H, L = 1, 2, 500
    q, k, v = _raw((B, H, L, 64), (B, H, L, 64), dtype, seed=3)
    g = torch.Generator().manual_seed(4)
    do = torch.randn(B, H, L, 64, generator=g).to(dtype)
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = linear_attention(*leaves, feature_map="elu+1")
    o.backward(do.cuda())
    fq, fk = np64(_mapped(q)), np64(_mapped(k))
    ref = cf.dense_backward(fq, fk, np64(v), np64(do), 1.0 / L)
    assert_parity(o, ref["o"], dtype, "o")
    # d phi(x)/dx = 1 for x > 0, exp(x) otherwise
    dphi = lambda x: np.where(np64(x) > 0, 1.0, np.exp(np.minimum(np64(x), 0.0)))
    assert_parity(leaves[0].grad, ref["dq"] * dphi(q), dtype, "dq")
    assert_parity(leaves[1].grad, ref["dk"] * dphi(k), dtype, "dk")
    assert_parity(leaves[2].grad, ref["dv"], dtype, "dv")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("B,H,L", [(2, 3, 300), (1, 2, 77), (8, 16, 2048)])
def test_gradients_with_respect_to_the_raw_tensors_from_the_kernels(B, H, L, dtype):
    """64-wide 16-bit heads: the backward kernels multiply dq and dk by the map's derivative
    themselves; the result agrees with the map differentiated by autograd (the path other shapes
    take), and the simple_la family does the same through the C ABI's flag."""
    from flash_bla import _hip
    from flash_bla.ops.feature_map import elu_plus_one
    from flash_bla.ops.linear_attn.fused import LinearAttnFunction, linear_attention
    q, k, v = _raw((B, H, L, 64), (B, H, L, 64), dtype, seed=L + 1)
    do = torch.randn(B, H, L, 64, generator=torch.Generator().manual_seed(L)).to(dtype).cuda()
    a = [t.cuda().requires_grad_() for t in (q, k, v)]
    linear_attention(*a, feature_map="elu+1").backward(do)
    b = [t.cuda().requires_grad_() for t in (q, k, v)]
    LinearAttnFunction.apply(*elu_plus_one(b[0], b[1]), b[2], 1.0 / L, 1e-6).backward(do)
    # (the kernels round dq, dk once, the other path twice: a couple of last places of the type)
    close = 1e-2 if dtype == torch.bfloat16 else 2e-3
    for name, x, y in zip(("dq", "dk", "dv"), a, b):
        assert max_rel_err(x.grad, np64(y.grad)) < close, name
    # the C ABI's other form: q, k are the mapped tensors (a binding that kept them), gradients gated
    qm, km_ = elu_plus_one(q.cuda(), k.cuda())
    _, s, km = _hip.la_fwd(qm, km_, v.cuda(), None, None, 1.0 / L, 1e-6, _hip.NORMALIZE)
    dq, dk, dv, _, _ = _hip.la_bwd(qm, km_, v.cuda(), None, None, do, s, km, 1.0 / L, 1e-6,
                                   _hip.NORMALIZE | _hip.ELU1_GRAD)
    for name, x, y in zip(("dq", "dk", "dv"), (dq, dk, dv), b):
        assert max_rel_err(x, np64(y.grad)) < close, name + " from mapped tensors"
    # without the denominator (the simple_la family), from mapped and from raw tensors
    scale = 0.125
    _, s, km = _hip.la_fwd(qm, km_, v.cuda(), None, None, scale, 1e-6, 0)
    ref = cf.dense_backward(np64(qm), np64(km_), np64(v), np64(do), scale, 1e-6, False)
    gate = lambda m: np.minimum(np64(m), 1.0)
    for what, args, flags in (("mapped", (qm, km_), _hip.ELU1_GRAD),
                              ("raw", (q.cuda(), k.cuda()), _hip.ELU1_QK | _hip.ELU1_GRAD)):
        dq, dk, dv, _, _ = _hip.la_bwd(*args, v.cuda(), None, None, do, s, km, scale, 1e-6, flags)
        assert_parity(dq, ref["dq"] * gate(qm), dtype, f"simple dq from {what}", ref.get("dq_mag"))
        assert_parity(dk, ref["dk"] * gate(km_), dtype, f"simple dk from {what}", ref.get("dk_mag"))
        assert_parity(dv, ref["dv"], dtype, f"simple dv from {what}", ref.get("dv_mag"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("D", [64, 32])
def test_simple_la_with_the_feature_map(D, dtype):
    """simple_la(..., feature_map="elu+1"): forward and gradients against the oracle on the mapped
    tensors, for the head size the kernels map themselves and for one that is mapped first."""
    from flash_bla.ops.simple_la.fused import simple_la
    B, H, L = 2, 2, 700
    q, k, v = _raw((B, H, L, D), (B, H, L, D), dtype, seed=D, spread=1.0)
    do = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(8)).to(dtype)
    with torch.no_grad():
        o_inference = simple_la(q.cuda(), k.cuda(), v.cuda(), feature_map="elu+1")
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = simple_la(*leaves, feature_map="elu+1")
    o.backward(do.cuda())
    ref = cf.dense_backward(np64(_mapped(q)), np64(_mapped(k)), np64(v), np64(do), D ** -0.5, 1e-6, False)
    dphi = lambda x: np.where(np64(x) > 0, 1.0, np.exp(np.minimum(np64(x), 0.0)))
    assert_parity(o_inference, ref["o"], dtype, "o (inference)")
    assert_parity(o, ref["o"], dtype, "o")
    assert_parity(leaves[0].grad, ref["dq"] * dphi(q), dtype, "dq", ref.get("dq_mag"))
    assert_parity(leaves[1].grad, ref["dk"] * dphi(k), dtype, "dk", ref.get("dk_mag"))
    assert_parity(leaves[2].grad, ref["dv"], dtype, "dv", ref.get("dv_mag"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_packed_gradients_through_the_feature_map(dtype):
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    lens = [5, 300, 1, 64, 1000, 17, 0, 2049]
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32)
    T, H = int(cu[-1]), 3
    q, k, v = _raw((T, H, 64), (T, H, 64), dtype, seed=19)
    do = torch.randn(T, H, 64, generator=torch.Generator().manual_seed(2)).to(dtype)
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu.cuda(), max(lens), feature_map="elu+1")
    o.backward(do.cuda())
    ref = cf.varlen_backward(np64(_mapped(q)), np64(_mapped(k)), np64(v), np64(do), cu.numpy())
    dphi = lambda x: np.where(np64(x) > 0, 1.0, np.exp(np.minimum(np64(x), 0.0)))
    assert_parity(o, ref["o"], dtype, "o")
    assert_parity(leaves[0].grad, ref["dq"] * dphi(q), dtype, "dq", ref.get("dq_mag"))
    assert_parity(leaves[1].grad, ref["dk"] * dphi(k), dtype, "dk", ref.get("dk_mag"))
    assert_parity(leaves[2].grad, ref["dv"], dtype, "dv", ref.get("dv_mag"))


@pytest.mark.parametrize("D,dtype", [(32, torch.float16), (128, torch.bfloat16), (64, torch.float32), (48, torch.float16)])
def test_other_shapes_map_first(D, dtype):
    from flash_bla.ops.linear_attn.fused import linear_attention
    B, H, L = 2, 2, 333
    q, k, v = _raw((B, H, L, D), (B, H, L, D), dtype, seed=D)
    with torch.no_grad():
        o = linear_attention(q.cuda(), k.cuda(), v.cuda(), feature_map="elu+1")
    ref = cf.dense_forward(np64(_mapped(q)), np64(_mapped(k)), np64(v), 1.0 / L)[0]
    assert_parity(o, ref, dtype, f"D{D}")


def test_argument_and_flag_errors():
    from flash_bla import _hip
    from flash_bla.ops.linear_attn.fused import linear_attention
    q, k, v = (t.cuda() for t in _raw((1, 1, 64, 64), (1, 1, 64, 64), torch.float16, seed=1))
    with pytest.raises(ValueError):
        linear_attention(q, k, v, feature_map="relu")
    # the C ABI refuses the flag where the kernels do not implement it
    q32, k32, v32 = (t.cuda() for t in _raw((1, 1, 64, 32), (1, 1, 64, 32), torch.float16, seed=2))
    with pytest.raises(ValueError, match="feature map on load"):
        _hip.la_fwd(q32, k32, v32, None, None, 1.0, 1e-6, _hip.NORMALIZE | _hip.ELU1_QK)
    o, s, km = _hip.la_fwd(q, k, v, None, None, 1.0, 1e-6, _hip.NORMALIZE)
    with pytest.raises(ValueError, match="needs FBLA_ELU1_GRAD"):
        _hip.la_bwd(q, k, v, None, None, torch.ones_like(v), s, km, 1.0, 1e-6, _hip.NORMALIZE | _hip.ELU1_QK)
    with pytest.raises(ValueError, match="backward entry points"):
        _hip.la_fwd(q, k, v, None, None, 1.0, 1e-6, _hip.NORMALIZE | _hip.ELU1_GRAD)
    o32, s32, km32 = _hip.la_fwd(q32, k32, v32, None, None, 1.0, 1e-6, _hip.NORMALIZE)
    with pytest.raises(ValueError, match="gradients through the feature map"):
        _hip.la_bwd(q32, k32, v32, None, None, torch.ones_like(v32), s32, km32, 1.0, 1e-6,
                    _hip.NORMALIZE | _hip.ELU1_GRAD)
