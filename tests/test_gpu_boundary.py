"""Properties of the C-ABI boundary itself: work goes to the caller's stream and nowhere
else, nothing synchronises or allocates behind the caller's back (so the entry points can be
captured into a HIP graph), and the entry points are re-entrant across host threads."""
import threading

import pytest
import torch

from helpers import make_qkv

pytestmark = pytest.mark.gpu


def _ops():
    from flash_bla import _hip
    return _hip


def _step(hip, q, k, v, do, scale):
    o, s, km = hip.la_fwd(q, k, v, None, None, scale, 1e-6, hip.NORMALIZE)
    dq, dk, dv, _, _ = hip.la_bwd(q, k, v, None, None, do, s, km, scale, 1e-6, hip.NORMALIZE)
    return o, dq, dk, dv


@pytest.mark.parametrize("shape", [(2, 4, 1024, 64), (1, 2, 700, 128)])
def test_graph_capture_replays_match_eager(shape):
    """Forward + backward captured once, replayed four times on fresh inputs with eager work
    and synchronisations in between; every replay must equal the eager result bit for bit
    (the reductions are fixed-order)."""
    hip = _ops()
    dev = torch.device("cuda")
    B, H, L, D = shape
    scale = 1.0 / L
    static = [t.to(dev) for t in make_qkv(shape, shape, torch.float16, seed=1)[:4]]
    _step(hip, *static, scale)  # warm-up outside the capture (module load, LDS attributes)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = _step(hip, *static, scale)
    for seed in (2, 3, 4, 5):
        fresh = [t.to(dev) for t in make_qkv(shape, shape, torch.float16, seed=seed)[:4]]
        eager = [t.clone() for t in _step(hip, *fresh, scale)]
        torch.cuda.synchronize()
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("o", "dq", "dk", "dv"), outs, eager):
            assert torch.equal(a, b), f"replay with seed {seed}: {name} differs from the eager result"


def test_captured_step_through_autograd_matches_eager():
    """`flash_bla.utils.CapturedStep`: the operator's forward and backward through torch.autograd
    recorded into one HIP graph; replays on fresh inputs, with eager steps and synchronisations in
    between, equal the eager output and gradients bit for bit."""
    from flash_bla.ops.linear_attn.fused import linear_attention
    from flash_bla.utils import CapturedStep
    dev = torch.device("cuda")
    shape = (2, 4, 1024, 64)
    q, k, v, do = (t.to(dev) for t in make_qkv(shape, shape, torch.float16, seed=11)[:4])
    leaves = [t.clone().requires_grad_() for t in (q, k, v)]
    captured = CapturedStep(linear_attention, leaves, do)
    for seed in (12, 13, 14):
        fresh = [t.to(dev) for t in make_qkv(shape, shape, torch.float16, seed=seed)[:4]]
        eager_in = [t.clone().requires_grad_() for t in fresh[:3]]
        eager_out = linear_attention(*eager_in)
        eager_out.backward(fresh[3])
        torch.cuda.synchronize()
        out, grads = captured(fresh[:3], fresh[3])
        torch.cuda.synchronize()
        assert torch.equal(out, eager_out), f"seed {seed}: output"
        for name, g, leaf in zip(("dq", "dk", "dv"), grads, eager_in):
            assert torch.equal(g, leaf.grad), f"seed {seed}: {name}"


def test_side_stream_only():
    """Launched on a side stream while the default stream is busy: the result is complete once
    that side stream is synchronised, and equals the default-stream result."""
    hip = _ops()
    dev = torch.device("cuda")
    shape = (2, 4, 2048, 64)
    q, k, v, do = (t.to(dev) for t in make_qkv(shape, shape, torch.bfloat16, seed=9)[:4])
    ref = [t.clone() for t in _step(hip, q, k, v, do, 1.0 / 2048)]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    busy = torch.empty(64 << 20, dtype=torch.float32, device=dev)
    for _ in range(8):
        busy.normal_()  # keeps the default stream occupied
    with torch.cuda.stream(side):
        got = _step(hip, q, k, v, do, 1.0 / 2048)
    side.synchronize()
    for a, b in zip(got, ref):
        assert torch.equal(a, b)
    torch.cuda.synchronize()


def test_two_host_threads():
    """Two host threads, each with its own stream and problem, call the entry points at the
    same time (error text and profiling mask are per thread; there is no other mutable state)."""
    hip = _ops()
    dev = torch.device("cuda")
    shapes = [(2, 4, 1536, 64), (1, 8, 1000, 64)]
    inputs = [[t.to(dev) for t in make_qkv(s, s, torch.float16, seed=20 + i)[:4]] for i, s in enumerate(shapes)]
    refs = [[t.clone() for t in _step(hip, *inp, 1.0 / s[2])] for inp, s in zip(inputs, shapes)]
    torch.cuda.synchronize()
    results, errors = [None, None], []

    def work(i):
        try:
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(20):
                    out = _step(hip, *inputs[i], 1.0 / shapes[i][2])
            stream.synchronize()
            results[i] = out
        except Exception as exc:  # surfaced below: an exception in a thread would otherwise be lost
            errors.append(exc)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for got, ref in zip(results, refs):
        for a, b in zip(got, ref):
            assert torch.equal(a, b)


def test_error_is_per_thread_and_does_not_poison():
    """A rejected call reports through the return code / last-error text and leaves the library
    usable: the next valid call succeeds."""
    hip = _ops()
    dev = torch.device("cuda")
    L = hip.lib()
    rc = L.fbla_la_fwd(None, None, None, None, None, None, None, None, None, 0, 1, 1, 16, 64, 64, 0, 1,
                       1.0, 1e-6, None)
    assert rc < 0
    assert L.fbla_last_error().decode() != ""
    shape = (1, 2, 256, 64)
    q, k, v, do = (t.to(dev) for t in make_qkv(shape, shape, torch.float16, seed=3)[:4])
    o, *_ = _step(hip, q, k, v, do, 1.0 / 256)
    assert torch.isfinite(o).all()


def test_views_off_a_16_byte_boundary():
    """A contiguous view that starts 2 bytes into a buffer: the bindings copy it to aligned memory
    (the kernels move 16-byte pieces); the C entry point itself refuses such a pointer."""
    import ctypes
    from flash_bla import _hip
    from flash_bla.ops.linear_attn.fused import linear_attention
    B, H, L, D = 1, 2, 100, 64
    n = B * H * L * D
    bufs = [torch.rand(n + 8, device="cuda", dtype=torch.float16) + 0.5 for _ in range(3)]
    q, k, v = (b[1:1 + n].view(B, H, L, D) for b in bufs)
    assert q.data_ptr() % 16 != 0 and q.is_contiguous()
    ref = linear_attention(q.clone(), k.clone(), v.clone())
    leaves = [t.detach().requires_grad_() for t in (q, k, v)]
    out = linear_attention(*leaves)
    assert torch.equal(out, ref)
    out.backward(torch.ones_like(out))
    assert all(torch.isfinite(t.grad).all() for t in leaves)
    lib = _hip.lib()
    o = torch.empty(B, H, L, D, device="cuda", dtype=torch.float16)
    s = torch.empty(B, H, D, D, device="cuda")
    km = torch.empty(B, H, D, device="cuda")
    ws = torch.empty(lib.fbla_la_workspace_bytes(0, B, H, L, D, D, _hip.F16, _hip.NORMALIZE) + 16, device="cuda",
                     dtype=torch.uint8)
    rc = lib.fbla_la_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), None, None, o.data_ptr(), s.data_ptr(),
                         km.data_ptr(), ws.data_ptr(), ws.numel(), B, H, L, D, D, _hip.F16, _hip.NORMALIZE,
                         ctypes.c_float(0.01), ctypes.c_float(1e-6), None)
    assert rc == -1 and b"aligned" in lib.fbla_last_error()
