"""numpy float64 closed forms (forward and backward) for every operator family.

Test infrastructure only (see oracle/__init__.py).  One function covers the
dense families; flags select the variant:

  normalize=True , decoupled=False -> linear_attention  (linear_attn/fused.py)
  normalize=False                   -> simple_la         (simple_la/fused.py)
  normalize=True , decoupled=True  -> decoupled_la      (linear_attn/decoupled.py)

Arrays are [..., L, D]; leading dims are batch/head.
"""
import numpy as np


def _f64(x):
    return np.asarray(x, dtype=np.float64)


def dense_forward(q, k, v, scale, eps=1e-6, normalize=True, q_rope=None, k_rope=None):
    """State S = scale * K~^T V, km = mean(K), z = q.km + eps, o = (q~ S)/z.

    linear_attn/fused.py:66-75,143-155; decoupled.py:81-83,171-180;
    simple_la/fused.py:61-69 (no denominator)."""
    q, k, v = _f64(q), _f64(k), _f64(v)
    qn = q if q_rope is None else _f64(q_rope)
    kn = k if k_rope is None else _f64(k_rope)
    S = scale * np.swapaxes(kn, -1, -2) @ v
    km = k.mean(axis=-2)
    if normalize:
        z = np.einsum('...ld,...d->...l', q, km) + eps
    else:
        z = np.ones(q.shape[:-1])
    o = (qn @ S) / z[..., None]
    return o, S, km, z


def dense_backward(q, k, v, do, scale, eps=1e-6, normalize=True, q_rope=None, k_rope=None):
    """Hand-derived gradients.

    dz_t = -(o_t.dO_t)/z_t, dS = sum_t (q~_t/z_t)^T dO_t, dkm = sum_t dz_t q_t,
    dq~_t = dO_t S^T / z_t, dq_t = dz_t km, dk~_t = scale v_t dS^T, dk_t = dkm/L,
    dv_t = scale k~_t dS   (linear_attn/fused.py:238-242,325-328;
    decoupled.py:274-283,375-380; simple_la/fused.py:198,394-397).
    Returns a dict with dq, dk, dv (+ dq_rope, dk_rope when decoupled).

    dq_mag / dk_mag give, element by element, the larger of the two terms that
    are added to form dq / dk.  For very short sequences the terms cancel (with
    L = 1 the output does not depend on q at all, up to eps), so a comparison of
    dq or dk should use max(|ref|.max(), mag.max()) as its scale."""
    decoupled = q_rope is not None
    q, k, v, do = _f64(q), _f64(k), _f64(v), _f64(do)
    qn = q if not decoupled else _f64(q_rope)
    kn = k if not decoupled else _f64(k_rope)
    L = k.shape[-2]
    o, S, km, z = dense_forward(q, k, v, scale, eps, normalize, q_rope, k_rope)
    zi = 1.0 / z[..., None]
    dS = np.swapaxes(qn * zi, -1, -2) @ do
    dq_num = (do @ np.swapaxes(S, -1, -2)) * zi
    dk_num = scale * (v @ np.swapaxes(dS, -1, -2))
    dv = scale * (kn @ dS)
    if normalize:
        dz = -(o * do).sum(-1, keepdims=True) * zi
        dq_den = dz * km[..., None, :]
        dkm = (dz * q).sum(axis=-2)
        dk_den = np.broadcast_to(dkm[..., None, :] / L, k.shape)
    else:
        dq_den = np.zeros_like(q)
        dk_den = np.zeros_like(k)
    if decoupled:
        return dict(dq=dq_den, dk=np.array(dk_den), dq_rope=dq_num, dk_rope=dk_num, dv=dv, o=o, S=S, km=km)
    return dict(dq=dq_num + dq_den, dk=dk_num + dk_den, dv=dv, o=o, S=S, km=km,
                dq_mag=np.maximum(np.abs(dq_num), np.abs(dq_den)),
                dk_mag=np.maximum(np.abs(dk_num), np.abs(dk_den)))


def varlen_forward(q, k, v, cu_seqlens, scale=None, eps=1e-6):
    """Per-sequence linear attention on packed [T,H,D] arrays; default scale is
    1/len_i per sequence (varlen.py:66,276)."""
    q, k, v = _f64(q), _f64(k), _f64(v)
    o = np.zeros(v.shape)
    cu = [int(x) for x in np.asarray(cu_seqlens).tolist()]
    for b, e in zip(cu[:-1], cu[1:]):
        if e <= b:
            continue
        s = 1.0 / (e - b) if scale is None else scale
        oi = dense_forward(q[b:e].transpose(1, 0, 2), k[b:e].transpose(1, 0, 2),
                           v[b:e].transpose(1, 0, 2), s, eps)[0]
        o[b:e] = oi.transpose(1, 0, 2)
    return o


def varlen_backward(q, k, v, do, cu_seqlens, scale=None, eps=1e-6):
    """varlen.py:216-219,310-314: the dense gradients applied per sequence."""
    q, k, v, do = _f64(q), _f64(k), _f64(v), _f64(do)
    out = dict(dq=np.zeros(q.shape), dk=np.zeros(k.shape), dv=np.zeros(v.shape), o=np.zeros(v.shape),
               dq_mag=np.zeros(q.shape), dk_mag=np.zeros(k.shape))
    cu = [int(x) for x in np.asarray(cu_seqlens).tolist()]
    for b, e in zip(cu[:-1], cu[1:]):
        if e <= b:
            continue
        s = 1.0 / (e - b) if scale is None else scale
        g = dense_backward(q[b:e].transpose(1, 0, 2), k[b:e].transpose(1, 0, 2),
                           v[b:e].transpose(1, 0, 2), do[b:e].transpose(1, 0, 2), s, eps)
        for name in ('dq', 'dk', 'dv', 'o', 'dq_mag', 'dk_mag'):
            out[name][b:e] = g[name].transpose(1, 0, 2)
    return out
