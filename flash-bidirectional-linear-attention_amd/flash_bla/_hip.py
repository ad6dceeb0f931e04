"""ctypes binding of libfbla_hip.so (declared in include/flash_bla_hip.h).

PyTorch is used for device memory (outputs, state, workspace come from its
caching allocator) and for the current stream; all arithmetic happens inside the
library.  There is no fallback: a missing library or a non-GPU tensor raises.
"""
import ctypes
import os

import torch

# FBLA_LIB_PATH selects another build of the library (A/B comparisons of kernel changes).
_LIB_PATH = os.environ.get("FBLA_LIB_PATH") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "_lib", "libfbla_hip.so")
_lib = None

F16, BF16, F32 = 0, 1, 2
NORMALIZE, DECOUPLED, DEFAULT_SCALE, ELU1_QK, ELU1_GRAD = 1, 2, 4, 8, 16

_DTYPES = {torch.float16: F16, torch.bfloat16: BF16, torch.float32: F32}

_vp, _i64, _i32, _f32, _sz = (ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float,
                              ctypes.c_size_t)

_SIGNATURES = {
    "fbla_version": (ctypes.c_int, []),
    "fbla_last_error": (ctypes.c_char_p, []),
    "fbla_set_phase_mask": (None, [ctypes.c_uint]),
    "fbla_la_workspace_bytes": (_sz, [_i32, _i64, _i64, _i64, _i32, _i32, _i32, _i32]),
    "fbla_la_fwd": (_i32, [_vp] * 9 + [_sz, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_static_scratch_bytes": (_sz, []),
    "fbla_la_fwd_static": (_i32, [_vp] * 8 + [_i64, _i64, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_la_bwd": (_i32, [_vp] * 14 + [_sz, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_la_pair_workspace_bytes": (_sz, [_i32, _i64, _i64, _i64, _i32, _i32, _i32]),
    "fbla_la_pair_fwd": (_i32, [_vp] * 9 + [_sz, _i64, _i64, _i64, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_la_pair_bwd": (_i32, [_vp] * 13 + [_sz, _i64, _i64, _i64, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_la_cross_workspace_bytes": (_sz, [_i32, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _i32]),
    "fbla_la_cross_fwd": (_i32, [_vp] * 7 + [_sz, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_la_cross_bwd": (_i32, [_vp] * 10 + [_sz, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_decoupled_cross_fwd": (_i32, [_vp] * 9 + [_sz, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_decoupled_cross_bwd": (_i32, [_vp] * 14 + [_sz, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_varlen_workspace_bytes": (_sz, [_i32, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _i32]),
    "fbla_varlen_fwd": (_i32, [_vp] * 8 + [_sz, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_varlen_bwd": (_i32, [_vp] * 11 + [_sz, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _f32, _f32, _vp]),
    "fbla_chunk_reduce_workspace_bytes": (_sz, [_i64, _i64, _i32, _i32, _i32, _i32, _i32]),
    "fbla_chunk_reduce": (_i32, [_vp] * 9 + [_sz, _i64, _i64, _i32, _i32, _i32, _f32, _i32, _vp]),
    "fbla_select_blocks": (_i32, [_vp] * 4 + [_i64, _i64, _i32, _i32, _f32, _vp]),
    "fbla_piecewise_workspace_bytes": (_sz, [_i64, _i64, _i32, _i32, _i32, _i32]),
    "fbla_piecewise_fwd": (_i32, [_vp] * 9 + [_sz, _i64, _i64, _i32, _i32, _i32, _i32, _f32, _i32, _vp]),
    "fbla_elu1_fwd": (_i32, [_vp, _vp, _i64, _vp, _vp, _i64, _i32, _vp]),
    "fbla_elu1_bwd": (_i32, [_vp, _vp, _vp, _i64, _i32, _vp]),
}


def lib_path():
    return _LIB_PATH


def exported_symbols():
    """Names this binding expects the shared library to export."""
    return sorted(_SIGNATURES)


def lib():
    """Load libfbla_hip.so once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError(
                f"flash_bla: HIP library not found at {_LIB_PATH}; build it with "
                "`make -C flash-bidirectional-linear-attention_amd/csrc` (there is no fallback path)")
        handle = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def _check(rc, what):
    if rc != 0:
        msg = lib().fbla_last_error().decode("utf-8", "replace")
        exc = ValueError if rc in (-1, -2) else RuntimeError
        raise exc(f"{what} failed ({rc}): {msg}")


def dtype_code(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError("q, k, and v must have dtype float16, bfloat16, or float32") from None


def _ptr(t):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device):
    """Handle of torch's current stream on `device` (the raw getter saves the Stream object: these
    wrappers are on the host-bound path of small problems)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class _Here:
    """No-op context: the tensors' device is already the current one."""
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_HERE = _Here()


_one_device = None


def _on(device):
    """Context that makes `device` current for the launch (kernels run on the current device).
    With a single visible GPU there is nothing to switch (and asking torch for the current device
    costs 2 us on the host-bound path of small problems)."""
    global _one_device
    if _one_device is None:
        _one_device = torch.cuda.device_count() == 1
    if _one_device or device.index is None or device.index == torch.cuda.current_device():
        return _HERE
    return torch.cuda.device(device)


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def _aligned(*tensors):
    """The kernels move 16-byte pieces: a tensor whose storage offset leaves its first element off
    a 16-byte boundary (a view into a larger buffer) is copied to fresh, aligned memory."""
    return tuple(t if t is None or t.data_ptr() % 16 == 0 else t.clone(memory_format=torch.contiguous_format)
                 for t in tensors)


def _require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise ValueError("flash_bla HIP operators need GPU tensors (got a CPU tensor); "
                             "use the naive_* functions for CPU math")


def la_fwd(q, k, v, q_rope, k_rope, scale, eps, flags):
    """Dense forward: returns (o, s, km).  Tensors must be contiguous [B,H,L,D]; k and v may have
    another number of tokens than q (not with the decoupled operator)."""
    _require_gpu(q, k, v, q_rope, k_rope)
    q, k, v, q_rope, k_rope = _aligned(q, k, v, q_rope, k_rope)
    L = lib()
    B, H, T, DK = q.shape
    Tk, DV = k.shape[-2], v.shape[-1]
    code = dtype_code(q)
    dev = q.device
    o = torch.empty(B, H, T, DV, dtype=v.dtype, device=dev)
    s = torch.empty(B, H, DK, DV, dtype=torch.float32, device=dev)
    km = torch.empty(B, H, DK, dtype=torch.float32, device=dev)
    if Tk != T and flags & DECOUPLED:
        with _on(dev):
            ws = _workspace(L.fbla_la_cross_workspace_bytes(0, B, H, T, Tk, DK, DV, code, flags), dev)
            rc = L.fbla_decoupled_cross_fwd(_ptr(q), _ptr(k), _ptr(q_rope), _ptr(k_rope), _ptr(v), _ptr(o), _ptr(s),
                                            _ptr(km), _ptr(ws), ws.numel(), B, H, T, Tk, DK, DV, code, float(scale),
                                            float(eps), _stream(dev))
        _check(rc, "fbla_decoupled_cross_fwd")
        return o, s, km
    if Tk != T:
        with _on(dev):
            ws = _workspace(L.fbla_la_cross_workspace_bytes(0, B, H, T, Tk, DK, DV, code, flags), dev)
            rc = L.fbla_la_cross_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(s), _ptr(km), _ptr(ws),
                                     ws.numel(), B, H, T, Tk, DK, DV, code, flags, float(scale), float(eps),
                                     _stream(dev))
        _check(rc, "fbla_la_cross_fwd")
        return o, s, km
    with _on(dev):
        ws = _workspace(L.fbla_la_workspace_bytes(0, B, H, T, DK, DV, code, flags), dev)
        rc = L.fbla_la_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(q_rope), _ptr(k_rope), _ptr(o), _ptr(s),
                           _ptr(km), _ptr(ws), ws.numel(), B, H, T, DK, DV, code, flags,
                           float(scale), float(eps), _stream(dev))
    _check(rc, "fbla_la_fwd")
    return o, s, km


def la_bwd(q, k, v, q_rope, k_rope, do, s, km, scale, eps, flags):
    """Dense backward: returns (dq, dk, dv, dq_rope, dk_rope)."""
    _require_gpu(q, k, v, do)
    q, k, v, q_rope, k_rope, do, s, km = _aligned(q, k, v, q_rope, k_rope, do, s, km)
    L = lib()
    B, H, T, DK = q.shape
    Tk, DV = k.shape[-2], v.shape[-1]
    code = dtype_code(q)
    dev = q.device
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    dqr = torch.empty_like(q_rope) if flags & DECOUPLED else None
    dkr = torch.empty_like(k_rope) if flags & DECOUPLED else None
    if Tk != T and flags & DECOUPLED:
        with _on(dev):
            ws = _workspace(L.fbla_la_cross_workspace_bytes(1, B, H, T, Tk, DK, DV, code, flags), dev)
            rc = L.fbla_decoupled_cross_bwd(_ptr(q), _ptr(k), _ptr(q_rope), _ptr(k_rope), _ptr(v), _ptr(do), _ptr(s),
                                            _ptr(km), _ptr(dq), _ptr(dk), _ptr(dqr), _ptr(dkr), _ptr(dv), _ptr(ws),
                                            ws.numel(), B, H, T, Tk, DK, DV, code, float(scale), float(eps),
                                            _stream(dev))
        _check(rc, "fbla_decoupled_cross_bwd")
        return dq, dk, dv, dqr, dkr
    if Tk != T:
        with _on(dev):
            ws = _workspace(L.fbla_la_cross_workspace_bytes(1, B, H, T, Tk, DK, DV, code, flags), dev)
            rc = L.fbla_la_cross_bwd(_ptr(q), _ptr(k), _ptr(v), _ptr(do), _ptr(s), _ptr(km), _ptr(dq),
                                     _ptr(dk), _ptr(dv), _ptr(ws), ws.numel(), B, H, T, Tk, DK, DV, code,
                                     flags, float(scale), float(eps), _stream(dev))
        _check(rc, "fbla_la_cross_bwd")
        return dq, dk, dv, None, None
    with _on(dev):
        ws = _workspace(L.fbla_la_workspace_bytes(1, B, H, T, DK, DV, code, flags), dev)
        rc = L.fbla_la_bwd(_ptr(q), _ptr(k), _ptr(v), _ptr(q_rope), _ptr(k_rope), _ptr(do), _ptr(s),
                           _ptr(km), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(dqr), _ptr(dkr), _ptr(ws),
                           ws.numel(), B, H, T, DK, DV, code, flags, float(scale), float(eps),
                           _stream(dev))
    _check(rc, "fbla_la_bwd")
    return dq, dk, dv, dqr, dkr


def pair_supported(q, v):
    """Whether the two-query operator covers these shapes (contiguous [B,H,L,DK] / [B,H,L,DV])."""
    B, H, T, DK = q.shape
    return bool(q.is_cuda and q.dtype in (torch.float16, torch.bfloat16) and
                lib().fbla_la_pair_workspace_bytes(0, B, H, T, DK, v.shape[-1], dtype_code(q)))


def pair_fwd(q1, q2, k, v, scale, eps):
    """Two queries on shared keys and values: returns (o1, o2, s, km); o_i are [B,H,L,DV/2]."""
    _require_gpu(q1, q2, k, v)
    q1, q2, k, v = _aligned(q1, q2, k, v)
    L = lib()
    B, H, T, DK = q1.shape
    DV = v.shape[-1]
    code = dtype_code(q1)
    dev = q1.device
    o1 = torch.empty(B, H, T, DV // 2, dtype=v.dtype, device=dev)
    o2 = torch.empty_like(o1)
    s = torch.empty(B, H, DK, DV, dtype=torch.float32, device=dev)
    km = torch.empty(B, H, DK, dtype=torch.float32, device=dev)
    with _on(dev):
        ws = _workspace(L.fbla_la_pair_workspace_bytes(0, B, H, T, DK, DV, code), dev)
        rc = L.fbla_la_pair_fwd(_ptr(q1), _ptr(q2), _ptr(k), _ptr(v), _ptr(o1), _ptr(o2), _ptr(s), _ptr(km),
                                _ptr(ws), ws.numel(), B, H, T, DK, DV, code, float(scale), float(eps), _stream(dev))
    _check(rc, "fbla_la_pair_fwd")
    return o1, o2, s, km


def pair_bwd(q1, q2, k, v, do1, do2, s, km, scale, eps):
    """Backward of pair_fwd: returns (dq1, dq2, dk, dv)."""
    _require_gpu(q1, q2, k, v, do1, do2)
    q1, q2, k, v, do1, do2, s, km = _aligned(q1, q2, k, v, do1, do2, s, km)
    L = lib()
    B, H, T, DK = q1.shape
    DV = v.shape[-1]
    code = dtype_code(q1)
    dev = q1.device
    dq1, dq2, dk, dv = torch.empty_like(q1), torch.empty_like(q2), torch.empty_like(k), torch.empty_like(v)
    with _on(dev):
        ws = _workspace(L.fbla_la_pair_workspace_bytes(1, B, H, T, DK, DV, code), dev)
        rc = L.fbla_la_pair_bwd(_ptr(q1), _ptr(q2), _ptr(k), _ptr(v), _ptr(do1), _ptr(do2), _ptr(s), _ptr(km),
                                _ptr(dq1), _ptr(dq2), _ptr(dk), _ptr(dv), _ptr(ws), ws.numel(), B, H, T, DK, DV,
                                code, float(scale), float(eps), _stream(dev))
    _check(rc, "fbla_la_pair_bwd")
    return dq1, dq2, dk, dv


def varlen_fwd(q, k, v, cu_seqlens, max_seqlen, scale, eps, extra_flags=0):
    """Packed forward: returns (o, s, km).  Tensors contiguous [T,H,D]."""
    _require_gpu(q, k, v, cu_seqlens)
    q, k, v, cu_seqlens = _aligned(q, k, v, cu_seqlens)
    L = lib()
    T, H, DK = q.shape
    DV = v.shape[-1]
    N = cu_seqlens.numel() - 1
    code = dtype_code(q)
    dev = q.device
    flags = NORMALIZE | (DEFAULT_SCALE if scale is None else 0) | extra_flags
    o = torch.empty_like(v)
    s = torch.empty(N, H, DK, DV, dtype=torch.float32, device=dev)
    km = torch.empty(N, H, DK, dtype=torch.float32, device=dev)
    with _on(dev):
        ws = _workspace(L.fbla_varlen_workspace_bytes(0, T, N, H, max_seqlen, DK, DV, code, flags), dev)
        rc = L.fbla_varlen_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(cu_seqlens), _ptr(o), _ptr(s),
                               _ptr(km), _ptr(ws), ws.numel(), T, N, H, max_seqlen, DK, DV, code,
                               flags, 0.0 if scale is None else float(scale), float(eps),
                               _stream(dev))
    _check(rc, "fbla_varlen_fwd")
    return o, s, km


def varlen_bwd(q, k, v, cu_seqlens, max_seqlen, do, s, km, scale, eps, extra_flags=0):
    """Packed backward: returns (dq, dk, dv)."""
    _require_gpu(q, k, v, do, cu_seqlens)
    q, k, v, do, cu_seqlens, s, km = _aligned(q, k, v, do, cu_seqlens, s, km)
    L = lib()
    T, H, DK = q.shape
    DV = v.shape[-1]
    N = cu_seqlens.numel() - 1
    code = dtype_code(q)
    dev = q.device
    flags = NORMALIZE | (DEFAULT_SCALE if scale is None else 0) | extra_flags
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    with _on(dev):
        ws = _workspace(L.fbla_varlen_workspace_bytes(1, T, N, H, max_seqlen, DK, DV, code, flags), dev)
        rc = L.fbla_varlen_bwd(_ptr(q), _ptr(k), _ptr(v), _ptr(cu_seqlens), _ptr(do), _ptr(s),
                               _ptr(km), _ptr(dq), _ptr(dk), _ptr(dv), _ptr(ws), ws.numel(), T, N,
                               H, max_seqlen, DK, DV, code, flags,
                               0.0 if scale is None else float(scale), float(eps), _stream(dev))
    _check(rc, "fbla_varlen_bwd")
    return dq, dk, dv


def chunk_reduce(q, k, v, chunk, with_norm=False, p_norm=2.0):
    """Block statistics of piecewise attention.  q,k:[B,H,T,K] v:[B,H,T,V] contiguous.
    Returns fp32 (qc, kc, vc, h, h_norm or None)."""
    _require_gpu(q, k, v)
    q, k, v = _aligned(q, k, v)
    L = lib()
    B, H, T, K = k.shape
    V = v.shape[-1]
    NT = -(-T // chunk)
    code = dtype_code(q)
    dev = q.device
    f32 = dict(dtype=torch.float32, device=dev)
    qc, kc = torch.empty(B, H, NT, K, **f32), torch.empty(B, H, NT, K, **f32)
    vc, h = torch.empty(B, H, NT, V, **f32), torch.empty(B, H, K, V, **f32)
    h_norm = torch.empty(B, H, NT, **f32) if with_norm else None
    with _on(dev):
        ws = _workspace(L.fbla_chunk_reduce_workspace_bytes(B * H, T, K, V, chunk, code, int(with_norm)), dev)
        rc = L.fbla_chunk_reduce(_ptr(q), _ptr(k), _ptr(v), _ptr(qc), _ptr(kc), _ptr(vc), _ptr(h),
                                 _ptr(h_norm), _ptr(ws), ws.numel(), B * H, T, K, V, chunk,
                                 float(p_norm), code, _stream(dev))
    _check(rc, "fbla_chunk_reduce")
    return qc, kc, vc, h, h_norm


def select_blocks(qc, kc, bias, top_k, scale):
    """Indices (int32, ascending) of the top_k key blocks per query block; qc, kc fp32 [B,H,NT,K]."""
    _require_gpu(qc, kc, bias)
    qc, kc, bias = _aligned(qc, kc, bias)
    L = lib()
    B, H, NT, K = qc.shape
    dev = qc.device
    idx = torch.empty(B, H, NT, top_k, dtype=torch.int32, device=dev)
    with _on(dev):
        rc = L.fbla_select_blocks(_ptr(qc), _ptr(kc), _ptr(bias), _ptr(idx), B * H, NT, K, top_k,
                                  float(scale), _stream(dev))
    _check(rc, "fbla_select_blocks")
    return idx


def piecewise_supported(q, v, block):
    B, H, T, K = q.shape
    return bool(q.dtype in _DTYPES and
                lib().fbla_piecewise_workspace_bytes(B * H, T, K, v.shape[-1], block, dtype_code(q)))


def piecewise_fwd(q, k, v, kc, vc, h, indices, block, scale):
    """Piecewise attention forward; indices int32 [B,H,NT,NS]; kc, vc, h fp32 from chunk_reduce."""
    _require_gpu(q, k, v, kc, vc, h, indices)
    q, k, v, kc, vc, h, indices = _aligned(q, k, v, kc, vc, h, indices)
    L = lib()
    B, H, T, K = q.shape
    V = v.shape[-1]
    NS = indices.shape[-1]
    code = dtype_code(q)
    dev = q.device
    o = torch.empty_like(v)
    with _on(dev):
        ws = _workspace(L.fbla_piecewise_workspace_bytes(B * H, T, K, V, block, code), dev)
        rc = L.fbla_piecewise_fwd(_ptr(q), _ptr(k), _ptr(v), _ptr(kc), _ptr(vc), _ptr(h), _ptr(indices),
                                  _ptr(o), _ptr(ws), ws.numel(), B * H, T, K, V, block, NS,
                                  float(scale), code, _stream(dev))
    _check(rc, "fbla_piecewise_fwd")
    return o


def elu1_fwd(x0, x1=None):
    """elu(x) + 1 of one or two contiguous tensors in one launch: returns the new tensor(s)."""
    _require_gpu(x0, x1)
    x0, x1 = _aligned(x0, x1)
    L = lib()
    y0 = torch.empty_like(x0)
    y1 = torch.empty_like(x1) if x1 is not None else None
    if x1 is not None and (x1.dtype != x0.dtype or x1.device != x0.device):
        raise ValueError("elu1_fwd: both tensors must have the same dtype and device")
    with _on(x0.device):
        rc = L.fbla_elu1_fwd(_ptr(x0), _ptr(y0), x0.numel(), _ptr(x1), _ptr(y1),
                             x1.numel() if x1 is not None else 0, dtype_code(x0), _stream(x0.device))
    _check(rc, "fbla_elu1_fwd")
    return y0 if x1 is None else (y0, y1)


def elu1_bwd(x, dy):
    """dy * d(elu(x) + 1)/dx for contiguous tensors of the same shape and dtype."""
    _require_gpu(x, dy)
    x, dy = _aligned(x, dy)
    L = lib()
    dx = torch.empty_like(x)
    with _on(x.device):
        rc = L.fbla_elu1_bwd(_ptr(x), _ptr(dy), _ptr(dx), x.numel(), dtype_code(x), _stream(x.device))
    _check(rc, "fbla_elu1_bwd")
    return dx
