"""Keys and values with another number of tokens than the queries (dense operators): the
PVT-style blocks reduce k, v spatially (`sr_ratio > 1`), the reference's kernels take one
length from q and run out of bounds there (linear_attn/fused.py:355).  Forward and backward
against the float64 oracle, on the matrix-core kernels and on the shape-generic ones."""
import pytest
import torch

from helpers import make_qkv, np64, parity_errors
from oracle import closed_form as cf

pytestmark = pytest.mark.gpu

LENGTHS = [(256, 64), (64, 256), (1000, 37), (5, 300), (3000, 750), (1, 8), (9000, 2250)]


def _check(variant, B, H, lq, lk, DK, DV, dtype, seed):
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.simple_la.fused import simple_la
    q, _, _, do = make_qkv((B, H, lq, DK), (B, H, lq, DV), dtype, seed)
    _, k, v, _ = make_qkv((B, H, lk, DK), (B, H, lk, DV), dtype, seed + 1)
    normalize = variant == "linear"
    scale = 1.0 / lk if normalize else DK ** -0.5
    ref = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), scale, 1e-6, normalize)
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = (linear_attention if normalize else simple_la)(*leaves)
    assert o.shape == (B, H, lq, DV) and o.dtype == dtype
    o.backward(do.cuda())
    errs = {"o": parity_errors(o, ref["o"], dtype)}
    for name, t in zip(("dq", "dk", "dv"), leaves):
        assert t.grad.shape == t.shape
        errs[name] = parity_errors(t.grad, ref[name], dtype, ref.get(name + "_mag"))
    bad = {n: e for n, e in errs.items() if not e[2]}
    assert not bad, f"{variant} {dtype} B{B} H{H} Lq{lq} Lk{lk} DK{DK} DV{DV}: {errs}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dims", [(64, 64), (32, 32), (128, 128), (128, 32), (64, 128), (48, 72)])
def test_linear_attention_16bit(dims, dtype):
    for i, (lq, lk) in enumerate(LENGTHS):
        _check("linear", 2, 3, lq, lk, dims[0], dims[1], dtype, 50 * i + dims[0])


@pytest.mark.parametrize("dims", [(64, 64), (32, 32), (128, 128), (64, 16)])
def test_simple_la_16bit(dims):
    for i, (lq, lk) in enumerate(LENGTHS[:5]):
        _check("simple", 1, 2, lq, lk, dims[0], dims[1], torch.float16, 70 * i + dims[1])


def test_fp32():
    for i, (lq, lk) in enumerate(LENGTHS):
        _check("linear", 2, 2, lq, lk, 64, 64, torch.float32, 90 + i)
        _check("linear", 1, 2, lq, lk, 32, 32, torch.float32, 190 + i)
    _check("simple", 1, 2, 300, 77, 64, 64, torch.float32, 99)
    _check("simple", 1, 2, 300, 77, 48, 20, torch.float32, 98)
    _check("linear", 2, 1, 77, 300, 12, 64, torch.float32, 97)


def test_default_scale_is_one_over_the_number_of_keys():
    from flash_bla.ops.linear_attn.fused import linear_attention
    q, _, _, _ = make_qkv((1, 2, 40, 64), (1, 2, 40, 64), torch.float16, 1)
    _, k, v, _ = make_qkv((1, 2, 10, 64), (1, 2, 10, 64), torch.float16, 2)
    a = linear_attention(q.cuda(), k.cuda(), v.cuda())
    b = linear_attention(q.cuda(), k.cuda(), v.cuda(), scale=0.1)
    assert torch.equal(a, b)


def test_shapes_of_the_generic_kernels():
    """Head dims that are not multiples of 8 (4 in fp32) and fp32 heads above 64 run on the
    shape-generic kernels, with another number of keys than queries as well."""
    for i, (lq, lk) in enumerate(LENGTHS[:4]):
        _check("linear", 1, 2, lq, lk, 20, 20, torch.float16, 300 + i)
        _check("linear", 2, 1, lq, lk, 17, 13, torch.bfloat16, 310 + i)
        _check("simple", 1, 2, lq, lk, 100, 36, torch.float16, 320 + i)
        _check("linear", 1, 2, lq, lk, 128, 128, torch.float32, 330 + i)
        _check("linear", 1, 1, lq, lk, 128, 32, torch.float32, 340 + i)
        _check("simple", 1, 2, lq, lk, 6, 70, torch.float32, 350 + i)


def _check_decoupled(B, H, lq, lk, DK, DV, dtype, seed):
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    q, _, _, do, qr = make_qkv((B, H, lq, DK), (B, H, lq, DV), dtype, seed, n_extra=1)
    _, k, v, _, kr = make_qkv((B, H, lk, DK), (B, H, lk, DV), dtype, seed + 1, n_extra=1)
    ref = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), 1.0 / lk, 1e-6, True, q_rope=np64(qr), k_rope=np64(kr))
    leaves = [t.cuda().requires_grad_() for t in (q, k, qr, kr, v)]
    o = decoupled_la(*leaves)
    assert o.shape == (B, H, lq, DV) and o.dtype == dtype
    o.backward(do.cuda())
    errs = {"o": parity_errors(o, ref["o"], dtype)}
    for name, t in zip(("dq", "dk", "dq_rope", "dk_rope", "dv"), leaves):
        assert t.grad.shape == t.shape
        errs[name] = parity_errors(t.grad, ref[name], dtype, ref.get(name + "_mag"))
    bad = {n: e for n, e in errs.items() if not e[2]}
    assert not bad, f"decoupled {dtype} B{B} H{H} Lq{lq} Lk{lk} DK{DK} DV{DV}: {errs}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=str)
@pytest.mark.parametrize("dims", [(32, 32), (64, 64), (128, 128), (64, 128), (20, 12)])
def test_decoupled_operator(dims, dtype):
    """Rotary and plain rows come in pairs of equal length on either side; the row-constant dk is
    dkm over the number of keys."""
    for i, (lq, lk) in enumerate(LENGTHS[:5]):
        _check_decoupled(1, 2, lq, lk, dims[0], dims[1], dtype, 400 + 10 * i + dims[0])


def test_decoupled_operator_shape_errors():
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    q64 = torch.rand(1, 2, 40, 64, device="cuda", dtype=torch.float16)
    k64 = torch.rand(1, 2, 10, 64, device="cuda", dtype=torch.float16)
    with pytest.raises(ValueError, match="shaped like"):
        decoupled_la(q64, k64, q64, q64, k64)     # k_rope with the queries' length
    with pytest.raises(ValueError, match="matching batch"):
        decoupled_la(q64, k64, q64, k64, q64)     # v with the queries' length
