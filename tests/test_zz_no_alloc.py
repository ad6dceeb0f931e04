"""The entry point that allocates nothing (fbla_la_fwd_static): called through the C ABI, its
output, state and mean key must equal those of fbla_la_fwd (same kernels, library-owned
scratch instead of a caller workspace) bit for bit, on two calls in a row with the second
input smaller than the first, and against the float64 oracle within the operator's gate."""
import pytest
import torch

from helpers import assert_parity, make_qkv, np64

pytestmark = pytest.mark.gpu


def _call_static(hip, q, k, v, scale, eps, flags):
    L = hip.lib()
    B, H, T, DK = q.shape
    DV = v.shape[-1]
    o = torch.empty_like(v)
    s = torch.empty(B, H, DK, DV, dtype=torch.float32, device=q.device)
    km = torch.empty(B, H, DK, dtype=torch.float32, device=q.device)
    rc = L.fbla_la_fwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), None, None, o.data_ptr(),
                              s.data_ptr(), km.data_ptr(), B, H, T, DK, DV, hip.dtype_code(q), flags,
                              scale, eps, torch.cuda.current_stream().cuda_stream)
    return rc, o, s, km


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_static_forward_equals_workspace_forward_twice(dtype):
    from flash_bla import _hip as hip
    from oracle import closed_form as cf
    dev = torch.device("cuda")
    # the first problem is split over several chunks per head (partials in the scratch), the
    # second is smaller and reuses the scratch the first one left behind
    for shape in ((2, 4, 6000, 64), (1, 3, 777, 64)):
        B, H, T, D = shape
        q, k, v, _ = make_qkv(shape, shape, dtype, seed=T)
        qd, kd, vd = (t.to(dev) for t in (q, k, v))
        need = hip.lib().fbla_la_workspace_bytes(0, B, H, T, D, D, hip.dtype_code(qd), hip.NORMALIZE)
        assert need <= hip.lib().fbla_static_scratch_bytes()
        print(f"static forward {dtype} {shape}: workspace {need} bytes", flush=True)
        rc, o, s, km = _call_static(hip, qd, kd, vd, 1.0 / T, 1e-6, hip.NORMALIZE)
        assert rc == 0, hip.lib().fbla_last_error()
        o_ref, s_ref, km_ref = hip.la_fwd(qd, kd, vd, None, None, 1.0 / T, 1e-6, hip.NORMALIZE)
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref) and torch.equal(s, s_ref) and torch.equal(km, km_ref)
        assert_parity(o, cf.dense_forward(np64(q), np64(k), np64(v), 1.0 / T)[0], dtype, "o")


def test_static_forward_rejects_oversized_problem():
    from flash_bla import _hip as hip
    dev = torch.device("cuda")
    L = hip.lib()
    # 4096 heads of 128x128: the per-chunk partials alone are far beyond the scratch
    B, H, T, D = 64, 64, 1 << 16, 128
    need = L.fbla_la_workspace_bytes(0, B, H, T, D, D, hip.F16, hip.NORMALIZE)
    if need <= L.fbla_static_scratch_bytes():
        pytest.skip("no dense shape here exceeds the scratch")
    x = torch.zeros(16, device=dev, dtype=torch.float16)
    f = torch.zeros(16, device=dev, dtype=torch.float32)
    rc = L.fbla_la_fwd_static(x.data_ptr(), x.data_ptr(), x.data_ptr(), None, None, x.data_ptr(),
                              f.data_ptr(), f.data_ptr(), B, H, T, D, D, hip.F16, hip.NORMALIZE, 1.0, 1e-6,
                              torch.cuda.current_stream().cuda_stream)
    assert rc == -3
    assert b"built-in scratch" in L.fbla_last_error()
