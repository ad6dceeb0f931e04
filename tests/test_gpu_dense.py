"""GPU parity of the dense operators (linear_attention, simple_la, decoupled_la)
against the float64 oracle, through the Python operator layer -> C ABI -> HIP."""
import glob
import os

import numpy as np
import pytest
import torch

from helpers import TOL, assert_parity, make_qkv, max_rel_err, np64, parity_errors
from oracle import closed_form as cf

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DTYPES = [torch.float16, torch.bfloat16, torch.float32]


def _run(variant, tensors, scale, eps, dtype):
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.simple_la.fused import simple_la
    dev = [t.to("cuda").requires_grad_() for t in tensors[:-1]]
    do = tensors[-1].to("cuda")
    if variant == "linear":
        o = linear_attention(*dev, scale=scale, eps=eps)
    elif variant == "simple":
        o = simple_la(*dev, scale=scale)
    else:
        q, k, v, qr, kr = dev
        o = decoupled_la(q, k, qr, kr, v, scale=scale, eps=eps)
    assert o.dtype == dtype and o.shape == do.shape
    o.backward(do)
    torch.cuda.synchronize()
    return o, [t.grad for t in dev]


def _check_dense(variant, B, H, L, DK, DV, dtype, scale=None, eps=1e-6, seed=42):
    q, k, v, do, qr, kr = make_qkv((B, H, L, DK), (B, H, L, DV), dtype, seed, n_extra=2)
    normalize = variant != "simple"
    s = scale if scale is not None else (1.0 / L if normalize else DK ** -0.5)
    kw = dict(q_rope=np64(qr), k_rope=np64(kr)) if variant == "decoupled" else {}
    ref = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), s, eps, normalize, **kw)
    tensors = (q, k, v, qr, kr, do) if variant == "decoupled" else (q, k, v, do)
    o, grads = _run(variant, tensors, scale, eps, dtype)
    names = ["dq", "dk", "dv", "dq_rope", "dk_rope"] if variant == "decoupled" else ["dq", "dk", "dv"]
    errs = {"o": parity_errors(o, ref["o"], dtype)}
    for name, g in zip(names, grads):
        assert g is not None and g.dtype == dtype
        errs[name] = parity_errors(g, ref[name], dtype, ref.get(name + "_mag"))
    bad = {n: e for n, e in errs.items() if not e[2]}
    assert not bad, f"{variant} {dtype} B{B} H{H} L{L} DK{DK} DV{DV}: (plain, excess, ok) = {errs}"


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("variant", ["linear", "simple", "decoupled"])
@pytest.mark.parametrize("B,H,L,DK,DV", [
    (2, 4, 256, 64, 64),      # the common head shape
    (1, 2, 37, 16, 8),        # ragged L, small unequal dims
    (1, 3, 1, 8, 8),          # single token
    (2, 2, 100, 17, 13),      # non power-of-two dims
    (1, 2, 300, 128, 128),    # largest head dims
    (1, 2, 200, 128, 32),     # PolaFormer-like DK = 4 DV
    (1, 2, 200, 32, 64),
    (2, 3, 333, 64, 128),     # mixed 64 / 128 head dims (MFMA path)
    (2, 3, 333, 128, 64),
    (1, 4, 4100, 128, 128),   # several chunks per head at the largest head dims
    (4, 16, 256, 32, 32),     # MLLA / RALA self-test shape (layers/mlla.py:102-127)
    (1, 2, 777, 96, 80),      # both head dims padded to the 128-wide tiles, ragged length
    (2, 2, 2050, 128, 72),    # several chunks, value dim padded to 128
])
def test_dense_parity(variant, B, H, L, DK, DV, dtype):
    _check_dense(variant, B, H, L, DK, DV, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_cpu_reference_config(dtype):
    """BASELINE config 1 shape: B=2, H=4, T=1024, D=64 (linear_attn and simple_la)."""
    _check_dense("linear", 2, 4, 1024, 64, 64, dtype)
    _check_dense("simple", 2, 4, 1024, 64, 64, dtype)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32], ids=str)
def test_explicit_scale_and_eps(dtype):
    _check_dense("linear", 1, 2, 130, 64, 64, dtype, scale=0.02, eps=1e-4)
    _check_dense("decoupled", 1, 2, 130, 32, 32, dtype, scale=1 / 130, eps=1e-4)
    _check_dense("simple", 1, 2, 130, 64, 48, dtype, scale=0.5)


@pytest.mark.parametrize("path", sorted(p for p in glob.glob(os.path.join(GOLDEN, "*.npz")) if not os.path.basename(p).startswith("layer_")), ids=os.path.basename)
@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_golden_fixtures(path, dtype):
    d = np.load(path)
    if "cu_seqlens" in d:
        pytest.skip("packed fixture (covered in test_gpu_varlen.py)")
    s, eps, normalize, dec = d["meta"]
    if dtype == torch.bfloat16:
        pytest.skip("fixture inputs are fp16-valued; bf16 would re-round them")
    variant = "decoupled" if dec else ("linear" if normalize else "simple")
    t = {n: torch.from_numpy(d[n]).to(dtype) for n in ("q", "k", "v", "do")}
    if dec:
        tensors = (t["q"], t["k"], t["v"], torch.from_numpy(d["q_rope"]).to(dtype),
                   torch.from_numpy(d["k_rope"]).to(dtype), t["do"])
    else:
        tensors = (t["q"], t["k"], t["v"], t["do"])
    o, grads = _run(variant, tensors, float(s), float(eps), dtype)
    names = ["dq", "dk", "dv", "dq_rope", "dk_rope"] if dec else ["dq", "dk", "dv"]
    assert_parity(o, d["ref_o"], dtype, "o")
    for name, g in zip(names, grads):
        assert_parity(g, d["ref_" + name], dtype, name,
                      d["ref_" + name + "_mag"] if "ref_" + name + "_mag" in d else None)


def test_non_contiguous_inputs_and_output_layout():
    from flash_bla.ops.linear_attn.fused import linear_attention
    q, k, v, do = make_qkv((2, 64, 3, 32), (2, 64, 3, 32), torch.float16, 7)
    qt, kt, vt = (x.cuda().transpose(1, 2) for x in (q, k, v))      # [B,H,L,D] views
    o = linear_attention(qt, kt, vt)
    ref = cf.dense_forward(np64(qt), np64(kt), np64(vt), 1 / 64)[0]
    assert_parity(o, ref, torch.float16, "o")


def test_results_are_bitwise_reproducible():
    from flash_bla.ops.linear_attn.fused import linear_attention
    q, k, v, do = make_qkv((2, 4, 2000, 64), (2, 4, 2000, 64), torch.float16, 11)
    outs = []
    for _ in range(3):
        leaves = [x.cuda().requires_grad_() for x in (q, k, v)]
        o = linear_attention(*leaves)
        o.backward(do.cuda())
        outs.append([o.detach()] + [x.grad for x in leaves])
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert torch.equal(a, b)


def test_matches_autograd_of_torch_formula_on_gpu():
    """Same comparison the reference layers' self-tests make (layers/linfusion.py:116-141):
    the operator against the torch formula differentiated by autograd, ratio gate 0.06."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.ops.linear_attn.naive import naive_linear_attn
    from flash_bla.utils import assert_close
    q, k, v, do = (x.cuda() for x in make_qkv((2, 16, 4096, 64), (2, 16, 4096, 64), torch.float32, 3))
    a = [x.clone().requires_grad_() for x in (q, k, v)]
    b = [x.clone().requires_grad_() for x in (q, k, v)]
    o = linear_attention(*a)
    ref = naive_linear_attn(*b)
    o.backward(do)
    ref.backward(do)
    assert_close("o", ref, o, 0.06)
    for name, x, y in zip("qkv", b, a):
        assert_close("d" + name, x.grad, y.grad, 0.06)
        assert max_rel_err(y.grad, x.grad) < 1e-4


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("variant", ["linear", "simple"])
@pytest.mark.parametrize("L", [1, 5, 15, 16, 17, 31, 33, 47, 8200])
def test_matrix_core_paths_at_awkward_lengths(variant, L, dtype):
    """64 x 64 heads run on the MFMA kernels for all three dtypes; their token loops work in
    tiles of 16 and 32 tokens with a moved-back last tile and a checked path below one tile."""
    _check_dense(variant, 1, 3, L, 64, 64, dtype, seed=L)


def test_decoupled_takes_fp32_rotary_features_next_to_16bit_inputs():
    """RoPE modules return fp32 (layers/mlla.py:32-36 of the reference): the rotary tensors are
    rounded to the type of q, their gradients come back in fp32."""
    from flash_bla.ops.linear_attn.decoupled import decoupled_la
    q, k, v, do, qr, kr = make_qkv((2, 2, 300, 32), (2, 2, 300, 32), torch.float32, 5, n_extra=2)
    h = lambda t: t.half()
    ref = cf.dense_backward(np64(h(q)), np64(h(k)), np64(h(v)), np64(h(do)), 1.0 / 300, 1e-6, True,
                            q_rope=np64(h(qr)), k_rope=np64(h(kr)))
    leaves = [h(q).cuda().requires_grad_(), h(k).cuda().requires_grad_(), qr.cuda().requires_grad_(),
              kr.cuda().requires_grad_(), h(v).cuda().requires_grad_()]
    o = decoupled_la(*leaves)
    assert o.dtype == torch.float16
    o.backward(h(do).cuda())
    assert leaves[2].grad.dtype == torch.float32 and leaves[3].grad.dtype == torch.float32
    assert_parity(o, ref["o"], torch.float16, "o")
    for name, t in zip(("dq", "dk", "dq_rope", "dk_rope", "dv"), leaves):
        assert_parity(t.grad, ref[name], torch.float16, name, ref.get(name + "_mag"))
