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


def test_static_forward_under_graph_capture():
    """The use the entry point exists for: after one eager call (which looks up the scratch address and
    sets the kernels' LDS attributes, neither of which may happen inside a capture) the call is recorded
    into a HIP graph; every replay on fresh inputs equals fbla_la_fwd bit for bit."""
    from flash_bla import _hip as hip
    dev = torch.device("cuda")
    B, H, T, D = 2, 4, 6000, 64
    dtype = torch.float16
    q, k, v, _ = make_qkv((B, H, T, D), (B, H, T, D), dtype, seed=5)
    qd, kd, vd = (t.to(dev) for t in (q, k, v))
    L = hip.lib()
    o = torch.empty_like(vd)
    s = torch.empty(B, H, D, D, dtype=torch.float32, device=dev)
    km = torch.empty(B, H, D, dtype=torch.float32, device=dev)

    def call():
        return L.fbla_la_fwd_static(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), None, None, o.data_ptr(),
                                    s.data_ptr(), km.data_ptr(), B, H, T, D, D, hip.dtype_code(qd), hip.NORMALIZE,
                                    1.0 / T, 1e-6, torch.cuda.current_stream().cuda_stream)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert call() == 0, L.fbla_last_error()   # eager warm-up on the capturing stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = call()
    assert rc == 0, L.fbla_last_error()
    for seed in (11, 12, 13):
        qn, kn, vn, _ = make_qkv((B, H, T, D), (B, H, T, D), dtype, seed=seed)
        qd.copy_(qn.to(dev)), kd.copy_(kn.to(dev)), vd.copy_(vn.to(dev))
        o.zero_(), s.zero_(), km.zero_()
        graph.replay()
        torch.cuda.synchronize()
        o_ref, s_ref, km_ref = hip.la_fwd(qd, kd, vd, None, None, 1.0 / T, 1e-6, hip.NORMALIZE)
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref) and torch.equal(s, s_ref) and torch.equal(km, km_ref), f"replay {seed}"


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
