"""fp32 inputs with a head dim above 64 (the matrix-core kernels tiled 128 x 128): dense, packed,
with and without the denominator, other numbers of keys than queries, against the float64 oracle
at the fp32 gate (1e-5).  (128, 128) in fp32 is a shape of the reference's own test matrix,
tests/ops/test_varlen_linear_attn.py:15-18."""
import pytest
import torch

from helpers import assert_parity, make_qkv, np64
from oracle import closed_form as cf

pytestmark = pytest.mark.gpu
DT = torch.float32


def _dense(variant, B, H, L, DK, DV, seed, Lk=None):
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.simple_la.fused import simple_la
    Lk = L if Lk is None else Lk
    q, _, _, do = make_qkv((B, H, L, DK), (B, H, L, DV), DT, seed)
    _, k, v, _ = make_qkv((B, H, Lk, DK), (B, H, Lk, DV), DT, seed + 1)
    normalize = variant == "linear"
    scale = 1.0 / Lk if normalize else DK ** -0.5
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = (linear_attention if normalize else simple_la)(*leaves)
    o.backward(do.cuda())
    if Lk == L:
        ref = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), scale, 1e-6, normalize)
    else:
        import numpy as np
        qt, kt, vt, dot = (t.double().requires_grad_() for t in (q, k, v, do))
        S = scale * kt.transpose(-1, -2) @ vt
        z = (qt @ kt.mean(-2, keepdim=True).transpose(-1, -2) + 1e-6) if normalize else 1.0
        oo = (qt @ S) / z
        oo.backward(do.double())
        ref = dict(o=oo.detach().numpy(), dq=qt.grad.numpy(), dk=kt.grad.numpy(), dv=vt.grad.numpy())
    tag = f"{variant} B{B} H{H} L{L}/{Lk} DK{DK} DV{DV}"
    assert_parity(o, ref["o"], DT, "o " + tag)
    for name, t in zip(("dq", "dk", "dv"), leaves):
        assert_parity(t.grad, ref[name], DT, f"{name} {tag}", ref.get(name + "_mag"))


@pytest.mark.parametrize("variant", ["linear", "simple"])
@pytest.mark.parametrize("B,H,L,DK,DV", [
    (2, 3, 777, 128, 128),    # the full tile
    (1, 2, 5000, 128, 128),   # several chunks per head: partials and their reduction
    (2, 2, 300, 96, 72),      # padded both ways
    (1, 3, 333, 128, 32),     # value blocks in the padding
    (1, 2, 450, 20, 100),     # key blocks in the padding
    (1, 1, 9, 68, 68),        # shorter than a tile
    (1, 2, 16, 128, 64),
    (1, 1, 1, 128, 128),      # one token
])
def test_dense_fp32_wide(variant, B, H, L, DK, DV):
    _dense(variant, B, H, L, DK, DV, seed=L + DK + DV)


@pytest.mark.parametrize("Lq,Lk", [(300, 75), (64, 1000)])
def test_dense_fp32_wide_other_number_of_keys(Lq, Lk):
    _dense("linear", 1, 2, Lq, 128, 96, seed=Lq, Lk=Lk)


@pytest.mark.parametrize("DK,DV", [(128, 128), (72, 128), (128, 16)])
def test_packed_fp32_wide(DK, DV):
    from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
    lengths = [1, 700, 33, 2100, 64, 15, 16, 17]
    cu = torch.tensor([0] + list(torch.tensor(lengths).cumsum(0)), dtype=torch.int32)
    T, H = int(cu[-1]), 3
    q, k, v, do = make_qkv((T, H, DK), (T, H, DV), DT, DK + DV)
    leaves = [t.cuda().requires_grad_() for t in (q, k, v)]
    o = varlen_linear_attention(*leaves, cu.cuda(), max(lengths))
    o.backward(do.cuda())
    ref = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.numpy())
    assert_parity(o, ref["o"], DT, "o")
    for name, t in zip(("dq", "dk", "dv"), leaves):
        for b, e in zip(cu[:-1].tolist(), cu[1:].tolist()):
            floor = ref[name + "_mag"][b:e] if name + "_mag" in ref else None
            assert_parity(t.grad[b:e], ref[name][b:e], DT, f"{name}[{b}:{e}]", floor)


def test_fp32_wide_runs_on_the_matrix_cores():
    """The library reports matrix-core support through the workspace it asks for: the per-row scalars of
    the two-kernel backward pass A (two floats per token and head) are part of it only on that path."""
    from flash_bla import _hip
    L = _hip.lib()
    B, H, T, D = 2, 4, 4096, 128
    need = L.fbla_la_workspace_bytes(1, B, H, T, D, D, _hip.F32, _hip.NORMALIZE)
    assert need >= 2 * B * H * T * 4
