"""numpy float64 dense evaluation of piecewise (PISA) attention, forward only.

Test infrastructure only (see oracle/__init__.py).  Written from
flash_bla/ops/piecewise_attn/kernel.py; the reference ships neither a naive
implementation nor a test for this operator; this closed form is pinned by
softmax-attention special cases and by the independent per-token C evaluation
oracle/piecewise_tokens.c (tests/test_oracle.py, including a mutation check of
the first-order coefficient).  What is implemented is the kernel's mathematics
with one group:

  s_ij  = scale * q_i.k_j                    exact scores       (kernel.py:227-228)
  sb_ic = scale * q_i.kc_c                   block-mean scores  (kernel.py:250-251)
  G_i   = sum_{c not selected} exp(sb_ic) n_c                  (kernel.py:275-276)
  o_i   = [ sum_{j in selected blocks} exp(s_ij) v_j
            + sum_{c not selected} exp(sb_ic) vc_c
            + (G_i / T) * scale * (q_i H) ]
          / [ sum_{j in selected} exp(s_ij) + G_i ]             (kernel.py:279-292)

with kc_c the mean key of chunk c, vc_c the SUM of values of chunk c, n_c the
chunk length and H = sum_c (K_c - kc_c)^T V_c (kernel.py:105-118,176).  The
Triton kernel does not rescale its running G when the running maximum changes
between groups (kernel.py:263-276), which makes its result depend on the
autotuned group size; the consistent value above is what is computed here.
"""
import numpy as np


def chunk_reduce(q, k, v, chunk_size):
    """kernel.py:89-128,152-176.  q,k:[T,K] v:[T,V] (one head).
    Returns qc[NT,K], kc[NT,K], vc[NT,V], hc[NT,K,V], H[K,V], lens[NT]."""
    q, k, v = (np.asarray(a, dtype=np.float64) for a in (q, k, v))
    T = k.shape[0]
    NT = -(-T // chunk_size)
    qc = np.zeros((NT, q.shape[1]))
    kc = np.zeros((NT, k.shape[1]))
    vc = np.zeros((NT, v.shape[1]))
    hc = np.zeros((NT, k.shape[1], v.shape[1]))
    lens = np.zeros(NT)
    for c in range(NT):
        sl = slice(c * chunk_size, min(T, (c + 1) * chunk_size))
        n = sl.stop - sl.start
        lens[c] = n
        qc[c] = q[sl].sum(0) / n
        kc[c] = k[sl].sum(0) / n
        vc[c] = v[sl].sum(0)
        hc[c] = (k[sl] - kc[c]).T @ v[sl]
    return qc, kc, vc, hc, hc.sum(0), lens


def select_blocks(qc, kc, scale, density, hc=None, use_bias=False, p=2):
    """kernel.py:313-318 (+172-174 for the bias): top-k key chunks per query chunk."""
    NT = qc.shape[0]
    score = qc @ (kc * scale).T
    if use_bias:
        h_norm = np.linalg.norm(hc.reshape(NT, -1), ord=p, axis=-1)
        score = score + np.log(h_norm + 1e-5)[None, :]
        score = np.exp(score - score.max(-1, keepdims=True))
        score = score / score.sum(-1, keepdims=True)
    top_k = max(1, int(density * NT))
    return np.argsort(-score, axis=-1, kind="stable")[:, :top_k]


def piecewise_forward(q, k, v, indices, block_size=64, scale=None, first_order=True):
    """One head.  q,k:[T,K] v:[T,V]; indices:[NT,NS] selected key chunks per query chunk."""
    q, k, v = (np.asarray(a, dtype=np.float64) for a in (q, k, v))
    T, K = k.shape
    scale = K ** -0.5 if scale is None else scale
    qc, kc, vc, hc, H, lens = chunk_reduce(q, k, v, block_size)
    NT = kc.shape[0]
    o = np.zeros((T, v.shape[1]))
    for t in range(NT):
        rows = slice(t * block_size, min(T, (t + 1) * block_size))
        qi = q[rows]
        sel = np.zeros(NT, dtype=bool)
        sel[np.asarray(indices[t], dtype=np.int64)] = True
        tok_sel = np.repeat(sel, block_size)[:T]
        s_exact = scale * (qi @ k[tok_sel].T)
        s_mean = scale * (qi @ kc[~sel].T)
        m = np.maximum(s_exact.max(-1, initial=-np.inf), s_mean.max(-1, initial=-np.inf))[:, None]
        pe = np.exp(s_exact - m)
        pm = np.exp(s_mean - m)
        G = pm @ lens[~sel]
        num = pe @ v[tok_sel] + pm @ vc[~sel]
        if first_order:
            num = num + (qi @ H) * (G / T * scale)[:, None]
        o[rows] = num / (pe.sum(-1) + G)[:, None]
    return o
