"""Host-side checks that need no GPU: the C-ABI library loads and exports every
declared symbol, host-only entry points answer, argument validation raises the
reference's exception types, and the oracle reproduces the golden fixtures."""
import ctypes
import glob
import os
import re

import numpy as np
import pytest
import torch

from flash_bla import _hip
from flash_bla.ops.linear_attn.varlen import varlen_linear_attention
from flash_bla.ops.linear_attn.fused import linear_attention
from oracle import closed_form as cf

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")


def _declared_symbols():
    names = set()
    for path in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(path).read(), flags=re.S)
        names.update(re.findall(r"\b(fbla_\w+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    declared = _declared_symbols()
    assert len(declared) >= 8
    handle = ctypes.CDLL(_hip.lib_path())
    for name in declared:
        assert hasattr(handle, name), f"{name} declared in include/ but not exported"
    assert set(declared) == set(_hip.exported_symbols())


def test_host_only_entry_points():
    L = _hip.lib()
    assert L.fbla_version() >= 100
    fwd = L.fbla_la_workspace_bytes(0, 8, 16, 16384, 64, 64, _hip.F16, _hip.NORMALIZE)
    bwd = L.fbla_la_workspace_bytes(1, 8, 16, 16384, 64, 64, _hip.F16, _hip.NORMALIZE)
    assert 0 < fwd <= bwd < (1 << 30)
    # workspace does not grow with L once the chunk count saturates
    assert L.fbla_la_workspace_bytes(0, 8, 16, 32768, 64, 64, _hip.F16, _hip.NORMALIZE) <= 2 * fwd
    assert L.fbla_varlen_workspace_bytes(0, 73000, 64, 16, 2048, 64, 64, _hip.BF16, 5) > 0


def test_skewed_packed_batches_reserve_partials_for_the_chunks_that_exist():
    """One sequence of 65536 tokens among 63 of 256 (H16, D128, bf16): the longest sequence is split
    into many chunks; the partial sums of the reductions get a slot per chunk that exists (at most
    T / chunk + N per head), not the long sequence's number of chunks for each of the 64 sequences."""
    L = _hip.lib()
    T, N, H = 65536 + 63 * 256, 64, 16
    slot = (128 * 128 + 128) * 4
    for which in (0, 1):
        need = L.fbla_varlen_workspace_bytes(which, T, N, H, 65536, 128, 128, _hip.BF16, 5)
        assert 0 < need < 160 * N * H * slot // 10   # well under 16 slots per (sequence, head)
    # an even batch keeps the plain layout and a small workspace
    assert L.fbla_varlen_workspace_bytes(0, 64 * 1200, 64, 16, 1200, 128, 128, _hip.BF16, 5) <= 2 * N * H * slot + 4096


def test_bad_arguments_return_error_codes_without_touching_the_gpu():
    L = _hip.lib()
    args = [None] * 9 + [0, 1, 1, 16, 0, 64, _hip.F16, _hip.NORMALIZE, 1.0, 1e-6, None]
    assert L.fbla_la_fwd(*args) == -2          # DK = 0
    assert b"head dims" in L.fbla_last_error()
    args[13:15] = [64, 64]
    args[15] = 7
    assert L.fbla_la_fwd(*args) == -1          # unknown dtype
    args[15], args[16] = _hip.F16, _hip.DECOUPLED
    assert L.fbla_la_fwd(*args) == -1          # decoupled without normalize
    args[16] = _hip.NORMALIZE
    assert L.fbla_la_fwd(*args) == -1          # null pointers with a non-empty problem
    assert b"null" in L.fbla_last_error()
    assert L.fbla_la_workspace_bytes(0, 1, 1, 16, 129, 64, 0, 1) == 0
    # the per-launch bits of the kernels' flag word are not the caller's to set
    for bits in (256, 512, 1024, _hip.NORMALIZE | 512):
        args[16] = bits
        assert L.fbla_la_fwd(*args) == -1
        assert b"unknown flag bits" in L.fbla_last_error()
        assert L.fbla_la_workspace_bytes(0, 1, 1, 16, 64, 64, _hip.F16, bits) == 0
        assert L.fbla_varlen_workspace_bytes(0, 1000, 4, 2, 512, 64, 64, _hip.F16, bits) == 0


def test_varlen_validation_matches_reference_exception_types():
    q = torch.rand(10, 2, 8)
    cu = torch.tensor([0, 4, 10], dtype=torch.int32)
    with pytest.raises(ValueError, match="shape"):
        varlen_linear_attention(q[0], q, q, cu, 6)
    with pytest.raises(ValueError, match="identical shapes"):
        varlen_linear_attention(q, q[:, :, :4], q, cu, 6)
    with pytest.raises(ValueError, match="matching token"):
        varlen_linear_attention(q, q, q[:5], cu, 6)
    with pytest.raises(ValueError, match="same dtype"):
        varlen_linear_attention(q, q, q.double(), cu, 6)
    with pytest.raises(ValueError, match="CUDA"):
        varlen_linear_attention(q, q, q, cu, 6)   # CPU tensors: no silent fallback


def test_dense_ops_refuse_cpu_tensors():
    q = torch.rand(1, 2, 8, 4)
    with pytest.raises(ValueError, match="GPU"):
        linear_attention(q, q, q)
    with pytest.raises(ValueError, match="must agree"):
        linear_attention(q, q[..., :2], q)
    with pytest.raises(ValueError, match="k and v"):
        linear_attention(q, q[:, :, :4], q)   # shorter keys are allowed, but v must follow k


def test_feature_map_refuses_cpu_tensors_and_bad_arguments():
    from flash_bla.ops.feature_map import elu_plus_one
    x = torch.rand(4, 8)
    with pytest.raises(ValueError, match="GPU"):
        elu_plus_one(x)                          # no CPU path behind the operator
    with pytest.raises(ValueError, match="same dtype"):
        elu_plus_one(x, x.double())
    with pytest.raises(TypeError):
        elu_plus_one(x.long())
    with pytest.raises(TypeError):
        elu_plus_one([1.0, 2.0])
    L = _hip.lib()
    assert L.fbla_elu1_fwd(None, None, -1, None, None, 0, _hip.F16, None) == -1   # negative size
    assert L.fbla_elu1_fwd(None, None, 8, None, None, 0, _hip.F16, None) == -1    # null pointers
    assert b"null" in L.fbla_last_error()
    assert L.fbla_elu1_fwd(None, None, 0, None, None, 0, 9, None) == -1           # unknown dtype
    assert L.fbla_elu1_bwd(None, None, None, 0, _hip.F32, None) == 0              # nothing to do
    assert L.fbla_elu1_fwd(None, None, 0, None, None, 0, _hip.BF16, None) == 0
    assert L.fbla_elu1_bwd(None, None, None, 5, _hip.F32, None) == -1


@pytest.mark.parametrize("path", sorted(p for p in glob.glob(os.path.join(GOLDEN, "*.npz")) if not os.path.basename(p).startswith("layer_")), ids=os.path.basename)
def test_oracle_reproduces_golden_fixture(path):
    d = np.load(path)
    if "cu_seqlens" in d:
        scale = None if d["meta"][0] < 0 else float(d["meta"][0])
        g = cf.varlen_backward(d["q"], d["k"], d["v"], d["do"], d["cu_seqlens"], scale, float(d["meta"][1]))
    else:
        s, eps, normalize, dec = d["meta"]
        kw = dict(q_rope=d["q_rope"], k_rope=d["k_rope"]) if dec else {}
        g = cf.dense_backward(d["q"], d["k"], d["v"], d["do"], float(s), float(eps), bool(normalize), **kw)
    for name, ref in d.items():
        if name.startswith("ref_") and name[4:] in g:
            got = g[name[4:]]
            if name.endswith("_mag"):
                got = got.max(axis=-1, keepdims=True)
            np.testing.assert_allclose(got, ref, rtol=1e-12, atol=1e-14)


def test_package_torch_formulas_match_the_oracle_restatement():
    """flash_bla.ops.*.naive are written in their own terms (one shared helper); the
    oracle restates the reference line by line.  Same values, fp64, all four functions."""
    import torch
    from flash_bla.ops.linear_attn import naive as pkg
    from flash_bla.ops.simple_la.naive import naive_simple_la
    from oracle import torch_ref as tr
    g = torch.Generator().manual_seed(3)
    q, k, qr, kr = (torch.rand(2, 3, 29, 12, generator=g, dtype=torch.float64) + 0.1 for _ in range(4))
    v = torch.randn(2, 3, 29, 7, generator=g, dtype=torch.float64)
    for scale in (None, 0.37):
        torch.testing.assert_close(pkg.naive_linear_attn(q, k, v, scale), tr.naive_linear_attn(q, k, v, scale),
                                   rtol=1e-12, atol=1e-14)
        torch.testing.assert_close(pkg.naive_decoupled_la(q, k, qr, kr, v, scale),
                                   tr.naive_decoupled_la(q, k, qr, kr, v, scale), rtol=1e-12, atol=1e-14)
        torch.testing.assert_close(naive_simple_la(q, k, v, scale), tr.naive_simple_la(q, k, v, scale),
                                   rtol=1e-12, atol=1e-14)
    cu = torch.tensor([0, 5, 18, 19, 40], dtype=torch.int32)
    qp, kp = (torch.rand(40, 3, 12, generator=g, dtype=torch.float64) + 0.1 for _ in range(2))
    vp = torch.randn(40, 3, 7, generator=g, dtype=torch.float64)
    for scale in (None, 0.2):
        torch.testing.assert_close(pkg.naive_varlen_linear_attn(qp, kp, vp, cu, scale, 1e-5),
                                   tr.naive_varlen_linear_attn(qp, kp, vp, cu, scale, 1e-5), rtol=1e-12, atol=1e-14)
