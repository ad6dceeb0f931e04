"""GPU parity of varlen_linear_attention: the reference's own test matrix
(tests/ops/test_varlen_linear_attn.py:11-55) plus layout equivalences."""
import glob
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from helpers import TOL, assert_parity, make_qkv, max_rel_err, np64
from oracle import closed_form as cf
from oracle import torch_ref as tr

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _cu(lengths, device="cuda"):
    return torch.tensor([0] + list(np.cumsum(lengths)), dtype=torch.int32, device=device)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=str)
@pytest.mark.parametrize("scale", [None, 0.02])
@pytest.mark.parametrize("heads", [1, 8])
@pytest.mark.parametrize(("key_dim", "value_dim"), [(8, 8), (17, 13), (64, 48), (128, 128)])
def test_varlen_linear_attention(dtype, scale, heads, key_dim, value_dim):
    """The reference's parametrised case, same seed, lengths, distributions and
    assert_close tolerances; the oracle stands in for naive_varlen_linear_attn."""
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    torch.manual_seed(42)
    lengths = [8, 17, 32]
    total = sum(lengths)
    cu = _cu(lengths)
    q = (F.elu(torch.randn(total, heads, key_dim, dtype=dtype, device="cuda")) + 1).requires_grad_()
    k = (F.elu(torch.randn(total, heads, key_dim, dtype=dtype, device="cuda")) + 1).requires_grad_()
    v = torch.randn(total, heads, value_dim, dtype=dtype, device="cuda", requires_grad=True)
    do = torch.randn_like(v)
    q_ref, k_ref, v_ref = (x.detach().clone().requires_grad_() for x in (q, k, v))

    out = varlen_linear_attention(q, k, v, cu, max(lengths), scale=scale)
    out_ref = tr.naive_varlen_linear_attn(q_ref, k_ref, v_ref, cu, scale=scale)
    out.backward(do)
    out_ref.backward(do)
    atol, rtol = (1e-5, 1e-4) if dtype == torch.float32 else (2e-2, 8e-2)
    torch.testing.assert_close(out, out_ref, atol=atol, rtol=rtol)
    torch.testing.assert_close(q.grad, q_ref.grad, atol=atol, rtol=rtol)
    torch.testing.assert_close(k.grad, k_ref.grad, atol=atol, rtol=rtol)
    torch.testing.assert_close(v.grad, v_ref.grad, atol=atol, rtol=rtol)
    # and the stricter gate against the float64 closed form
    g = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.cpu().numpy(), scale)
    assert_parity(out, g["o"], dtype, "o")
    for name, t in (("dq", q), ("dk", k), ("dv", v)):
        assert_parity(t.grad, g[name], dtype, name, g.get(name + "_mag"))


def test_varlen_linear_attention_oversized_max_seqlen():
    """tests/ops/test_varlen_linear_attn.py:45-55."""
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    lengths = [7, 11]
    cu = _cu(lengths)
    g = torch.Generator().manual_seed(0)
    q = torch.rand(sum(lengths), 2, 16, generator=g).cuda()
    k = torch.rand(sum(lengths), 2, 16, generator=g).cuda()
    v = torch.randn(sum(lengths), 2, 16, generator=g).cuda()
    expected = varlen_linear_attention(q, k, v, cu, max(lengths))
    oversized = varlen_linear_attention(q, k, v, cu, q.shape[0])
    torch.testing.assert_close(oversized, expected)
    assert torch.equal(oversized, expected)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=str)
@pytest.mark.parametrize("D", [64, 128])
def test_varlen_ragged_batch(dtype, D):
    """A scaled-down BASELINE config 3: ragged lengths, 16 heads, fwd + bwd."""
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    g = torch.Generator().manual_seed(42)
    lengths = torch.randint(1, 300, (9,), generator=g).tolist() + [1, 513]
    T = sum(lengths)
    q, k, v, do = make_qkv((T, 16, D), (T, 16, D), dtype, 5)
    cu = _cu(lengths)
    leaves = [x.cuda().requires_grad_() for x in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu, max(lengths))
    o.backward(do.cuda())
    ref = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.cpu().numpy())
    assert_parity(o, ref["o"], dtype, "o")
    for name, t in zip(("dq", "dk", "dv"), leaves):
        # gradients of different sequences differ in magnitude by their lengths:
        # compare sequence by sequence
        for b, e in zip(cu[:-1].tolist(), cu[1:].tolist()):
            floor = ref[name + "_mag"][b:e] if name + "_mag" in ref else None
            assert_parity(t.grad[b:e], ref[name][b:e], dtype, f"{name}[{b}:{e}]", floor)


def test_varlen_single_sequence_equals_dense():
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    q, k, v, do = (x.cuda() for x in make_qkv((333, 4, 64), (333, 4, 64), torch.float16, 9))
    cu = _cu([333])
    o = varlen_linear_attention(q, k, v, cu, 333)
    od = linear_attention(*(x.transpose(0, 1)[None] for x in (q, k, v)))
    assert max_rel_err(o, od[0].transpose(0, 1)) < 1e-3


def test_varlen_zero_length_sequence_is_skipped():
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    lengths = [5, 0, 9]
    q, k, v, do = make_qkv((14, 2, 16), (14, 2, 16), torch.float32, 13)
    cu = _cu(lengths)
    leaves = [x.cuda().requires_grad_() for x in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu, 9)
    o.backward(do.cuda())
    ref = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.cpu().numpy())
    assert max_rel_err(o, ref["o"]) <= 1e-5
    for name, t in zip(("dq", "dk", "dv"), leaves):
        assert torch.isfinite(t.grad).all()
        assert max_rel_err(t.grad, ref[name], ref.get(name + "_mag")) <= 1e-5


def test_varlen_rejects_bad_cu_seqlens_on_gpu():
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    q = torch.rand(10, 2, 8, device="cuda")
    with pytest.raises(ValueError, match="int32"):
        varlen_linear_attention(q, q, q, torch.tensor([0, 10], device="cuda"), 10)
    with pytest.raises(ValueError, match="positive integer"):
        varlen_linear_attention(q, q, q, _cu([10]), 0)
    with pytest.raises(TypeError):
        varlen_linear_attention(q.double(), q.double(), q.double(), _cu([10]), 10)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "varlen_*.npz"))), ids=os.path.basename)
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32], ids=str)
def test_varlen_golden_fixtures(path, dtype):
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    d = np.load(path)
    scale = None if d["meta"][0] < 0 else float(d["meta"][0])
    leaves = [torch.from_numpy(d[n]).to(dtype).cuda().requires_grad_() for n in ("q", "k", "v")]
    cu = torch.from_numpy(d["cu_seqlens"]).cuda()
    lens = np.diff(d["cu_seqlens"])
    o = varlen_linear_attention(*leaves, cu, int(lens.max()), scale=scale, eps=float(d["meta"][1]))
    o.backward(torch.from_numpy(d["do"]).to(dtype).cuda())
    assert_parity(o, d["ref_o"], dtype, "o")
    for name, t in zip(("dq", "dk", "dv"), leaves):
        for b, e in zip(d["cu_seqlens"][:-1], d["cu_seqlens"][1:]):
            floor = d["ref_" + name + "_mag"][b:e] if "ref_" + name + "_mag" in d else None
            assert_parity(t.grad[b:e], d["ref_" + name][b:e], dtype, name, floor)


@pytest.mark.parametrize("nseq", [128, 129, 1025, 3000])
def test_varlen_many_short_sequences(nseq):
    """Around and beyond the number of sequences whose lengths every workgroup ranks itself for
    the longest-first walk (128): beyond it a small kernel writes the order once per call."""
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    rng = np.random.default_rng(nseq)
    lengths = rng.integers(0, 40, nseq).tolist()
    lengths[7] = 900   # one long sequence among the short ones
    T, H, D = sum(lengths), 2, 64
    q, k, v, do = make_qkv((T, H, D), (T, H, D), torch.bfloat16, nseq)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32).cuda()
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu, max(lengths))
    o.backward(do.cuda())
    ref = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.cpu().numpy())
    assert_parity(o, ref["o"], torch.bfloat16, "o")
    # gradients sequence by sequence would be 3000 comparisons: compare the long one and the whole
    b, e = int(cu[7]), int(cu[8])
    for name, t in zip(("dq", "dk", "dv"), leaves):
        assert_parity(t.grad[b:e], ref[name][b:e], torch.bfloat16, f"{name} long", ref.get(name + "_mag", ref[name])[b:e])
        assert_parity(t.grad, ref[name], torch.bfloat16, name, ref.get(name + "_mag"))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=str)
@pytest.mark.parametrize("D", [64, 128, 32])
def test_varlen_one_long_sequence_among_short_ones(D, dtype):
    """A skewed batch: the long sequence is split over many workgroups (chunks that the short
    sequences do not have), its partial sums are reduced in chunk order."""
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    lengths = [20] * 17 + [9000] + [35] * 30 + [0, 1]
    T, H = sum(lengths), 3
    q, k, v, do = make_qkv((T, H, D), (T, H, D), dtype, D)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32).cuda()
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu, max(lengths))
    o.backward(do.cuda())
    ref = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.cpu().numpy())
    assert_parity(o, ref["o"], dtype, "o")
    for name, t in zip(("dq", "dk", "dv"), leaves):
        for b, e in zip(cu[:-1].tolist(), cu[1:].tolist()):
            if e > b:
                floor = ref[name + "_mag"][b:e] if name + "_mag" in ref else None
                assert_parity(t.grad[b:e], ref[name][b:e], dtype, f"{name}[{b}:{e}]", floor)


@pytest.mark.parametrize("nseq", [8, 9, 17, 40])
def test_varlen_sequences_dealt_to_the_xcds(nseq):
    """From eight sequences on, the row-parallel kernels deal the sequences out to the eight XCDs
    and walk a sequence's heads and chunks as consecutive workgroups of one XCD; sequences past the
    last multiple of eight keep the plain order.  Long sequences (several chunks each) next to
    short and empty ones."""
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    rng = np.random.default_rng(nseq)
    lengths = rng.integers(0, 300, nseq).tolist()
    lengths[1], lengths[nseq - 1], lengths[nseq // 2] = 7000, 2500, 0
    T, H, D, dtype = sum(lengths), 5, 64, torch.bfloat16
    q, k, v, do = make_qkv((T, H, D), (T, H, D), dtype, 300 + nseq)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32).cuda()
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu, max(lengths))
    o.backward(do.cuda())
    ref = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.cpu().numpy())
    assert_parity(o, ref["o"], dtype, "o")
    for name, t in zip(("dq", "dk", "dv"), leaves):
        for b, e in zip(cu[:-1].tolist(), cu[1:].tolist()):
            if e > b:
                floor = ref[name + "_mag"][b:e] if name + "_mag" in ref else None
                assert_parity(t.grad[b:e], ref[name][b:e], dtype, f"{name}[{b}:{e}]", floor)
