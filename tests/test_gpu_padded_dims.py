"""Head dims that are multiples of 8 but not 64 or 128 (the MLLA / RALA blocks use 32, the
PolaFormer block 2d x d/2) run on the matrix-core kernels with the last 64-wide block of a
head partly empty.  Forward and backward of every operator family against the float64
oracle, dense and packed, with sequence lengths that take the single-chunk path, the
path with several chunks per head, ragged tiles and one-token sequences."""
import numpy as np
import pytest
import torch

from helpers import assert_parity, make_qkv, np64, parity_errors
from oracle import closed_form as cf

pytestmark = pytest.mark.gpu

HEAD_DIMS = [(32, 32), (16, 16), (8, 8), (24, 40), (64, 32), (32, 64), (128, 32), (64, 16), (72, 72),
             (96, 128), (120, 8), (128, 104), (48, 48)]
LENGTHS = [1, 17, 300, 2500]


def _check_dense(variant, B, H, L, DK, DV, dtype, seed):
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.simple_la.fused import simple_la
    q, k, v, do, qr, kr = make_qkv((B, H, L, DK), (B, H, L, DV), dtype, seed, n_extra=2)
    normalize = variant != "simple"
    scale = 1.0 / L if normalize else DK ** -0.5
    kw = dict(q_rope=np64(qr), k_rope=np64(kr)) if variant == "decoupled" else {}
    ref = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), scale, 1e-6, normalize, **kw)
    tensors = (q, k, qr, kr, v) if variant == "decoupled" else (q, k, v)
    leaves = [t.cuda().requires_grad_() for t in tensors]
    op = {"linear": linear_attention, "simple": simple_la, "decoupled": decoupled_la}[variant]
    names = ["dq", "dk", "dq_rope", "dk_rope", "dv"] if variant == "decoupled" else ["dq", "dk", "dv"]
    o = op(*leaves)
    o.backward(do.cuda())
    errs = {"o": parity_errors(o, ref["o"], dtype)}
    for name, t in zip(names, leaves):
        errs[name] = parity_errors(t.grad, ref[name], dtype, ref.get(name + "_mag"))
    bad = {n: e for n, e in errs.items() if not e[2]}
    assert not bad, f"{variant} {dtype} B{B} H{H} L{L} DK{DK} DV{DV}: {errs}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dims", HEAD_DIMS)
def test_dense_linear_attention(dims, dtype):
    for i, L in enumerate(LENGTHS):
        _check_dense("linear", 2, 3, L, dims[0], dims[1], dtype, 10 * i + dims[0])


@pytest.mark.parametrize("dims", HEAD_DIMS)
def test_dense_simple_la(dims):
    for i, L in enumerate(LENGTHS[1:]):
        _check_dense("simple", 1, 2, L, dims[0], dims[1], torch.float16, 20 * i + dims[1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dims", [(32, 32), (16, 16), (8, 24), (64, 32), (40, 64), (96, 32)])
def test_dense_decoupled(dims, dtype):
    for i, L in enumerate(LENGTHS):
        _check_dense("decoupled", 2, 2, L, dims[0], dims[1], dtype, 30 * i + dims[0])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dims", [(32, 32), (16, 16), (48, 48), (96, 96), (32, 64), (128, 40), (8, 72)])
def test_packed(dims, dtype):
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    DK, DV = dims
    H = 5
    lengths = [300, 1, 0, 17, 1200, 64, 33]
    T = sum(lengths)
    q, k, v, do = make_qkv((T, H, DK), (T, H, DV), dtype, DK + DV)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32).cuda()
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu, max(lengths))
    o.backward(do.cuda())
    ref = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.cpu().numpy())
    tag = f"{dtype} DK{DK} DV{DV}"
    assert_parity(o, ref["o"], dtype, f"o {tag}")
    for name, t in zip(("dq", "dk", "dv"), leaves):
        for b, e in zip(cu[:-1].tolist(), cu[1:].tolist()):
            if e > b:
                floor = ref[name + "_mag"][b:e] if name + "_mag" in ref else None
                assert_parity(t.grad[b:e], ref[name][b:e], dtype, f"{name}[{b}:{e}] {tag}", floor)


def test_many_chunks_per_head():
    """One head, long sequence: several chunks per head in every kernel, partials summed by the
    consumers."""
    _check_dense("linear", 1, 1, 20000, 32, 32, torch.float16, 7)
    _check_dense("linear", 1, 1, 9000, 128, 32, torch.bfloat16, 8)
    _check_dense("decoupled", 1, 1, 9000, 32, 32, torch.float16, 9)


def test_heads_tiled_128_by_128():
    """The 128 x 128 backward kernel (eight waves share a step of 128 tokens): several chunks per
    head, lengths that leave one to three of a step's four tiles empty, the unnormalised
    operator, head dims below 128 in both tiles."""
    _check_dense("linear", 1, 1, 9000, 128, 128, torch.bfloat16, 11)
    _check_dense("linear", 2, 3, 33, 128, 128, torch.float16, 12)
    _check_dense("linear", 2, 3, 200, 128, 128, torch.bfloat16, 13)
    _check_dense("simple", 1, 2, 3000, 128, 128, torch.float16, 14)
    _check_dense("simple", 1, 2, 97, 128, 128, torch.bfloat16, 15)
    _check_dense("linear", 1, 1, 5000, 96, 120, torch.float16, 16)
    _check_dense("linear", 3, 2, 129, 72, 128, torch.bfloat16, 17)


@pytest.mark.parametrize("dims,dtype,L", [((128, 128), torch.bfloat16, 1030), ((96, 120), torch.float16, 1100),
                                           ((128, 72), torch.bfloat16, 2049)])
def test_whole_state_per_wave_dense(dims, dtype, L):
    """256 heads of more than 1024 tokens with a state tiled 128 x 128 (one workgroup per head in
    the state kernel, the row kernel and backward pass A for 128-wide heads).  A few heads are
    checked against the oracle."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    DK, DV = dims
    B, H = 16, 16
    g = torch.Generator().manual_seed(DK + L)
    q = (torch.nn.functional.elu(torch.randn(B, H, L, DK, generator=g)) + 1).to(dtype)
    k = (torch.nn.functional.elu(torch.randn(B, H, L, DK, generator=g)) + 1).to(dtype)
    v = torch.randn(B, H, L, DV, generator=g).to(dtype)
    do = torch.randn(B, H, L, DV, generator=g).to(dtype)
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = linear_attention(*leaves)
    o.backward(do.cuda())
    for b, h in ((0, 0), (7, 9), (15, 15)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        ref = cf.dense_backward(np64(q[sl]), np64(k[sl]), np64(v[sl]), np64(do[sl]), 1.0 / L, 1e-6, True)
        tag = f"{dtype} DK{DK} DV{DV} head ({b},{h})"
        assert_parity(o[sl], ref["o"], dtype, f"o {tag}")
        for name, t in zip(("dq", "dk", "dv"), leaves):
            assert_parity(t.grad[sl], ref[name], dtype, f"{name} {tag}", ref.get(name + "_mag"))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("dims", [(128, 128), (104, 96), (72, 128), (128, 32), (64, 128), (96, 48), (16, 120)])
def test_heads_tiled_128_around_the_64_token_steps(dims, dtype):
    """The kernels for heads tiled 128 x 128 walk steps of 64 tokens staged in LDS: lengths just
    below, at and above one, two and three steps, one chunk and several chunks per head.  Heads
    with one side of at most 64 take the same backward pass A (as padded 128 x 128 heads)."""
    for i, L in enumerate([63, 64, 65, 127, 128, 129, 191, 193, 640, 1153]):
        _check_dense("linear", 1, 2, L, dims[0], dims[1], dtype, 90 * i + dims[0])
    _check_dense("simple", 2, 1, 130, dims[0], dims[1], dtype, 7 + dims[1])
    _check_dense("linear", 2, 70, 321, dims[0], dims[1], dtype, 11 + dims[1])  # one chunk per head


def test_whole_state_per_wave_packed():
    """The same kernels on a packed batch: 320 (sequence, head) pairs, the longest sequence above
    1024 tokens, among them sequences shorter than one tile, of one token and empty ones."""
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    H, DK, DV, dtype = 8, 128, 128, torch.bfloat16
    lengths = [1500, 1024, 1, 0, 17, 2100, 15, 16, 33, 700] * 4
    T = sum(lengths)
    q, k, v, do = make_qkv((T, H, DK), (T, H, DV), dtype, 77)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32).cuda()
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu, max(lengths))
    o.backward(do.cuda())
    for h in (0, 5):
        hs = slice(h, h + 1)
        ref = cf.varlen_backward(np64(q[:, hs]), np64(k[:, hs]), np64(v[:, hs]), np64(do[:, hs]), cu.cpu().numpy())
        assert_parity(o[:, hs], ref["o"], dtype, f"o head {h}")
        for name, t in zip(("dq", "dk", "dv"), leaves):
            for b, e in zip(cu[:-1].tolist(), cu[1:].tolist()):
                if e > b:
                    floor = ref[name + "_mag"][b:e] if name + "_mag" in ref else None
                    assert_parity(t.grad[b:e, hs], ref[name][b:e], dtype, f"{name}[{b}:{e}] head {h}", floor)


@pytest.mark.parametrize("dims", [(32, 32), (16, 16), (4, 4), (24, 40), (64, 32), (32, 64), (60, 12), (48, 48)])
def test_fp32_head_dims_up_to_64(dims):
    """fp32 inputs: head dims that are multiples of 4 up to 64 run on the fp32 matrix instructions."""
    for i, L in enumerate(LENGTHS):
        _check_dense("linear", 2, 3, L, dims[0], dims[1], torch.float32, 40 * i + dims[0])
    _check_dense("simple", 1, 2, 700, dims[0], dims[1], torch.float32, 41 + dims[1])


def test_fp32_packed_small_heads():
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    for DK, DV in ((32, 32), (16, 48), (64, 8)):
        H = 3
        lengths = [300, 1, 0, 17, 1200, 64, 33]
        T = sum(lengths)
        q, k, v, do = make_qkv((T, H, DK), (T, H, DV), torch.float32, DK + DV)
        cu = torch.tensor(np.concatenate([[0], np.cumsum(lengths)]), dtype=torch.int32).cuda()
        leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
        o = varlen_linear_attention(*leaves, cu, max(lengths))
        o.backward(do.cuda())
        ref = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.cpu().numpy())
        assert_parity(o, ref["o"], torch.float32, f"o DK{DK} DV{DV}")
        for name, t in zip(("dq", "dk", "dv"), leaves):
            for b, e in zip(cu[:-1].tolist(), cu[1:].tolist()):
                if e > b:
                    floor = ref[name + "_mag"][b:e] if name + "_mag" in ref else None
                    assert_parity(t.grad[b:e], ref[name][b:e], torch.float32, f"{name}[{b}:{e}] DK{DK} DV{DV}", floor)


@pytest.mark.parametrize("dims", [(32, 32), (64, 64), (16, 40), (64, 32), (4, 60)])
def test_fp32_decoupled(dims):
    """The decoupled operator in fp32 (the MLLA / RALA blocks without autocast)."""
    for i, L in enumerate(LENGTHS + [5000]):
        _check_dense("decoupled", 2, 2, L, dims[0], dims[1], torch.float32, 60 * i + dims[1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=str)
@pytest.mark.parametrize("variant,DK,DV", [("linear", 100, 100), ("simple", 17, 13), ("decoupled", 30, 50),
                                           ("linear", 125, 7), ("linear", 3, 2)])
def test_head_dims_between_row_lengths_are_widened(variant, DK, DV, dtype):
    """Head dims that are not multiples of 8 (16-bit) / 4 (fp32) run on the matrix-core kernels through
    zero-widened workspace copies (the decoupled operator in fp32 only up to 64): same results as the
    original problem, checked against the float64 oracle like every other shape."""
    from flash_bla import _hip
    B, H, L = 2, 3, 333
    _check_dense(variant, B, H, L, DK, DV, dtype, DK * 7 + DV)
    # the workspace the library asks for holds the widened copies (the shape-generic path needs far less)
    code = {torch.float16: _hip.F16, torch.bfloat16: _hip.BF16, torch.float32: _hip.F32}[dtype]
    flags = _hip.NORMALIZE * (variant != "simple") | _hip.DECOUPLED * (variant == "decoupled")
    unit = 4 if dtype == torch.float32 else 8
    widened = (DK % unit or DV % unit) and not (dtype == torch.float32 and variant == "decoupled" and max(DK, DV) > 64)
    need = _hip.lib().fbla_la_workspace_bytes(0, B, H, L, DK, DV, code, flags)
    if widened:
        assert need >= 3 * B * H * L * min(DK, DV) * (4 if dtype == torch.float32 else 2)
