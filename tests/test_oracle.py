"""Pins the CPU oracle (oracle/) without a GPU.

The reference holds no golden vectors for these operators, so the oracle is
pinned by (i) an O(L^2) brute-force evaluation in plain C that never forms the
K^T V state, (ii) closed-form special cases and invariants, (iii) agreement of
the three independent restatements (torch formulas, float64 closed forms, C),
and (iv) torch.autograd / gradcheck for the hand-derived backward.
"""
import numpy as np
import pytest
import torch

from helpers import make_qkv, np64
from oracle import brute, closed_form as cf, piecewise as pw, torch_ref as tr
from oracle.piecewise_tokens import pisa_tokens


def _dense_inputs(B=2, H=3, L=37, DK=16, DV=8, seed=0, n_extra=0):
    return make_qkv((B, H, L, DK), (B, H, L, DV), torch.float64, seed, n_extra)


@pytest.mark.parametrize("L,DK,DV", [(1, 4, 3), (37, 16, 8), (64, 8, 24)])
@pytest.mark.parametrize("scale", [None, 0.37])
def test_linear_attn_matches_brute_force(L, DK, DV, scale):
    q, k, v, _ = _dense_inputs(1, 2, L, DK, DV)
    s = 1.0 / L if scale is None else scale
    o_cf = cf.dense_forward(np64(q), np64(k), np64(v), s)[0]
    o_tr = np64(tr.naive_linear_attn(q, k, v, scale))
    for h in range(2):
        o_b = brute.brute_linear_attn(np64(q)[0, h], np64(k)[0, h], np64(v)[0, h], s)
        np.testing.assert_allclose(o_cf[0, h], o_b, rtol=1e-12, atol=1e-13)
        np.testing.assert_allclose(o_tr[0, h], o_b, rtol=1e-11, atol=1e-12)


def test_simple_la_matches_brute_force():
    q, k, v, _ = _dense_inputs(1, 2, 29, 12, 20)
    o_tr = np64(tr.naive_simple_la(q, k, v))
    o_cf = cf.dense_forward(np64(q), np64(k), np64(v), 12 ** -0.5, normalize=False)[0]
    for h in range(2):
        o_b = brute.brute_linear_attn(np64(q)[0, h], np64(k)[0, h], np64(v)[0, h], 12 ** -0.5,
                                      normalize=False)
        np.testing.assert_allclose(o_tr[0, h], o_b, rtol=1e-11, atol=1e-12)
        np.testing.assert_allclose(o_cf[0, h], o_b, rtol=1e-12, atol=1e-13)
    # associativity: scale * (q k^T) v
    ref = (q @ k.transpose(-1, -2)) @ v * 12 ** -0.5
    np.testing.assert_allclose(o_tr, np64(ref), rtol=1e-11, atol=1e-12)


def test_decoupled_matches_brute_force_and_reduces_to_plain():
    q, k, v, _, qr, kr = _dense_inputs(1, 2, 33, 8, 8, n_extra=2)
    o_tr = np64(tr.naive_decoupled_la(q, k, qr, kr, v))
    o_cf = cf.dense_forward(np64(q), np64(k), np64(v), 1 / 33, q_rope=np64(qr), k_rope=np64(kr))[0]
    for h in range(2):
        o_b = brute.brute_linear_attn(np64(q)[0, h], np64(k)[0, h], np64(v)[0, h], 1 / 33,
                                      q_rope=np64(qr)[0, h], k_rope=np64(kr)[0, h])
        np.testing.assert_allclose(o_tr[0, h], o_b, rtol=1e-11, atol=1e-12)
        np.testing.assert_allclose(o_cf[0, h], o_b, rtol=1e-12, atol=1e-13)
    same = tr.naive_decoupled_la(q, k, q, k, v)
    np.testing.assert_allclose(np64(same), np64(tr.naive_linear_attn(q, k, v)), rtol=1e-13)


def test_invariants():
    q, k, v, _ = _dense_inputs(1, 1, 50, 8, 5)
    L = 50
    o = tr.naive_linear_attn(q, k, v)
    # constant v = c  =>  o = c * z / (z + eps) with z = q.km  (default scale 1/L)
    c = torch.full_like(v, 1.7)
    z = (q @ k.mean(-2, keepdim=True).transpose(-1, -2))
    np.testing.assert_allclose(np64(tr.naive_linear_attn(q, k, c)), np64(1.7 * z / (z + 1e-6)).repeat(5, -1),
                               rtol=1e-12)
    # joint permutation of (k, v) rows leaves o unchanged
    perm = torch.randperm(L, generator=torch.Generator().manual_seed(1))
    np.testing.assert_allclose(np64(tr.naive_linear_attn(q, k[..., perm, :], v[..., perm, :])), np64(o),
                               rtol=1e-11, atol=1e-13)
    # k -> a*k leaves o unchanged as eps -> 0
    np.testing.assert_allclose(np64(tr.naive_linear_attn(q, 3 * k, v, eps=0.0)),
                               np64(tr.naive_linear_attn(q, k, v, eps=0.0)), rtol=1e-11, atol=1e-13)
    # linear in v
    v2 = torch.randn(v.shape, dtype=v.dtype, generator=torch.Generator().manual_seed(2))
    np.testing.assert_allclose(np64(tr.naive_linear_attn(q, k, 2 * v - 3 * v2)),
                               np64(2 * o - 3 * tr.naive_linear_attn(q, k, v2)), rtol=1e-10, atol=1e-12)
    # every output component lies inside the range of the values (positive features)
    assert (o <= v.max(-2, keepdim=True).values + 1e-12).all()
    assert (o >= v.min(-2, keepdim=True).values - 1e-12).all()
    # L = 1, scale = 1:  o = v (q.k)/(q.k + eps)
    q1, k1, v1 = q[..., :1, :], k[..., :1, :], v[..., :1, :]
    qk = (q1 * k1).sum(-1, keepdim=True)
    np.testing.assert_allclose(np64(tr.naive_linear_attn(q1, k1, v1, scale=1.0)), np64(v1 * qk / (qk + 1e-6)),
                               rtol=1e-12)
    # the LinFusion layer's torch formula is linear_attn with eps = 1e-4
    np.testing.assert_allclose(np64(tr.linfusion_torch_mode(q, k, v)),
                               np64(tr.naive_linear_attn(q, k, v, eps=1e-4)), rtol=1e-11)


@pytest.mark.parametrize("variant", ["linear", "simple", "decoupled"])
def test_closed_form_backward_matches_autograd(variant):
    q, k, v, do, qr, kr = _dense_inputs(2, 2, 23, 8, 6, n_extra=2)
    leaves = [t.clone().requires_grad_() for t in (q, k, v, qr, kr)]
    ql, kl, vl, qrl, krl = leaves
    if variant == "linear":
        o = tr.naive_linear_attn(ql, kl, vl, 0.11)
        g = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), 0.11)
    elif variant == "simple":
        o = tr.naive_simple_la(ql, kl, vl, 0.11)
        g = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), 0.11, normalize=False)
    else:
        o = tr.naive_decoupled_la(ql, kl, qrl, krl, vl, 0.11)
        g = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), 0.11, q_rope=np64(qr),
                              k_rope=np64(kr))
    o.backward(do)
    np.testing.assert_allclose(g["o"], np64(o), rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(g["dq"], np64(ql.grad), rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(g["dk"], np64(kl.grad), rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(g["dv"], np64(vl.grad), rtol=1e-9, atol=1e-11)
    if variant == "decoupled":
        np.testing.assert_allclose(g["dq_rope"], np64(qrl.grad), rtol=1e-9, atol=1e-11)
        np.testing.assert_allclose(g["dk_rope"], np64(krl.grad), rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("normalize", [True, False])
def test_fewer_or_more_keys_than_queries(normalize):
    """k, v with another number of tokens than q (the PVT-style blocks shorten the keys): the
    closed form against the O(Lq Lk) double sum written out, and its gradients against autograd."""
    for lq, lk in ((23, 9), (5, 31)):
        q, _, _, do, _, _ = _dense_inputs(2, 2, lq, 8, 6, n_extra=2)
        _, k, v, _, _, _ = _dense_inputs(2, 2, lk, 8, 6, n_extra=2)
        scale, eps = 0.07, 1e-6
        g = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), scale, eps, normalize)
        w = np.einsum("bhik,bhjk->bhij", np64(q), np64(k))          # q_i . k_j
        num = scale * np.einsum("bhij,bhjv->bhiv", w, np64(v))
        ref = num / (w.mean(-1, keepdims=True) + eps) if normalize else num
        np.testing.assert_allclose(g["o"], ref, rtol=1e-11, atol=1e-13)
        ql, kl, vl = (t.clone().requires_grad_() for t in (q, k, v))
        o = tr.naive_linear_attn(ql, kl, vl, scale) if normalize else tr.naive_simple_la(ql, kl, vl, scale)
        o.backward(do)
        np.testing.assert_allclose(g["o"], np64(o), rtol=1e-11, atol=1e-13)
        for name, leaf in (("dq", ql), ("dk", kl), ("dv", vl)):
            np.testing.assert_allclose(g[name], np64(leaf.grad), rtol=1e-9, atol=1e-11)


def test_decoupled_with_fewer_or_more_keys_than_queries():
    """The decoupled closed form with Lq != Lk: output against the double sum written out
    (numerator from the rotary rows, denominator from the plain ones, mean over the Lk keys), all
    five gradients against autograd on the torch restatement."""
    for lq, lk in ((23, 9), (5, 31)):
        q, _, _, do, qr, _ = _dense_inputs(2, 2, lq, 8, 6, n_extra=2)
        _, k, v, _, _, kr = _dense_inputs(2, 2, lk, 8, 6, n_extra=2)
        scale, eps = 0.07, 1e-6
        g = cf.dense_backward(np64(q), np64(k), np64(v), np64(do), scale, eps, True, q_rope=np64(qr), k_rope=np64(kr))
        num = scale * np.einsum("bhij,bhjv->bhiv", np.einsum("bhik,bhjk->bhij", np64(qr), np64(kr)), np64(v))
        den = np.einsum("bhik,bhjk->bhij", np64(q), np64(k)).mean(-1, keepdims=True) + eps
        np.testing.assert_allclose(g["o"], num / den, rtol=1e-11, atol=1e-13)
        leaves = [t.clone().requires_grad_() for t in (q, k, qr, kr, v)]
        o = tr.naive_decoupled_la(*leaves, scale)
        o.backward(do)
        np.testing.assert_allclose(g["o"], np64(o), rtol=1e-11, atol=1e-13)
        for name, leaf in zip(("dq", "dk", "dq_rope", "dk_rope", "dv"), leaves):
            np.testing.assert_allclose(g[name], np64(leaf.grad), rtol=1e-9, atol=1e-11)


def test_gradcheck_torch_ref():
    q, k, v, _ = _dense_inputs(1, 1, 7, 3, 2)
    args = [t.clone().requires_grad_() for t in (q, k, v)]
    assert torch.autograd.gradcheck(lambda a, b, c: tr.naive_linear_attn(a, b, c, 0.3), args)
    assert torch.autograd.gradcheck(lambda a, b, c: tr.naive_simple_la(a, b, c, 0.3), args)


def _varlen_inputs(lengths, H=2, DK=8, DV=5, seed=3):
    T = int(sum(lengths))
    q, k, v, do = make_qkv((T, H, DK), (T, H, DV), torch.float64, seed)
    cu = torch.tensor([0] + list(np.cumsum(lengths)), dtype=torch.int32)
    return q, k, v, do, cu


@pytest.mark.parametrize("scale", [None, 0.02])
def test_varlen_equals_dense_per_sequence(scale):
    lengths = [8, 17, 32]
    q, k, v, do, cu = _varlen_inputs(lengths)
    o = tr.naive_varlen_linear_attn(q, k, v, cu, scale)
    o_cf = cf.varlen_forward(np64(q), np64(k), np64(v), cu.numpy(), scale)
    np.testing.assert_allclose(np64(o), o_cf, rtol=1e-11, atol=1e-13)
    for b, e in zip(cu[:-1].tolist(), cu[1:].tolist()):
        dense = tr.naive_linear_attn(q[b:e].transpose(0, 1)[None], k[b:e].transpose(0, 1)[None],
                                     v[b:e].transpose(0, 1)[None], scale)
        np.testing.assert_allclose(np64(o[b:e]), np64(dense[0].transpose(0, 1)), rtol=1e-11, atol=1e-13)
    # backward
    leaves = [t.clone().requires_grad_() for t in (q, k, v)]
    tr.naive_varlen_linear_attn(*leaves, cu, scale).backward(do)
    g = cf.varlen_backward(np64(q), np64(k), np64(v), np64(do), cu.numpy(), scale)
    for name, leaf in zip(("dq", "dk", "dv"), leaves):
        np.testing.assert_allclose(g[name], np64(leaf.grad), rtol=1e-9, atol=1e-11)


def test_varlen_equal_lengths_is_dense_batch():
    q, k, v, _, cu = _varlen_inputs([16, 16, 16])
    o = tr.naive_varlen_linear_attn(q, k, v, cu)
    qd, kd, vd = (t.view(3, 16, 2, -1).permute(0, 2, 1, 3) for t in (q, k, v))
    od = tr.naive_linear_attn(qd, kd, vd)
    np.testing.assert_allclose(np64(o), np64(od.permute(0, 2, 1, 3).reshape(48, 2, -1)), rtol=1e-12)


# ---------------------------------------------------------------------------
# piecewise (PISA) oracle: mathematical pins only (reference parity unpinned)
# ---------------------------------------------------------------------------
def _pw_inputs(T=200, K=16, V=8, seed=5):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(T, d, generator=g, dtype=torch.float64).numpy() for d in (K, K, V))


def test_piecewise_all_blocks_selected_is_softmax_attention():
    q, k, v = _pw_inputs()
    NT = -(-200 // 64)
    idx = np.tile(np.arange(NT), (NT, 1))
    o = pw.piecewise_forward(q, k, v, idx, 64)
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q)[None], torch.from_numpy(k)[None], torch.from_numpy(v)[None])[0].numpy()
    np.testing.assert_allclose(o, ref, rtol=1e-10, atol=1e-12)


def test_piecewise_constant_keys_per_chunk_zeroth_order_exact():
    # identical keys inside every chunk: block-mean scores are exact and H = 0,
    # so ANY selection reproduces softmax attention.
    q, k, v = _pw_inputs(T=192)
    k = np.repeat(k[::64], 64, axis=0)
    qc, kc, vc, hc, H, lens = pw.chunk_reduce(q, k, v, 64)
    assert np.abs(H).max() < 1e-12
    idx = np.array([[0], [2], [1]])
    o = pw.piecewise_forward(q, k, v, idx, 64)
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q)[None], torch.from_numpy(k)[None], torch.from_numpy(v)[None])[0].numpy()
    np.testing.assert_allclose(o, ref, rtol=1e-10, atol=1e-12)


def test_piecewise_chunk_reduce_and_selection():
    q, k, v = _pw_inputs(T=200)
    qc, kc, vc, hc, H, lens = pw.chunk_reduce(q, k, v, 64)
    assert lens.tolist() == [64, 64, 64, 8]
    np.testing.assert_allclose(kc[3], k[192:].mean(0))
    np.testing.assert_allclose(vc[3], v[192:].sum(0))
    np.testing.assert_allclose((kc * lens[:, None]).sum(0), k.sum(0), rtol=1e-12)
    # H = K^T V - sum_c n_c kc_c vc_c^T / n_c
    np.testing.assert_allclose(H, k.T @ v - np.einsum('ck,cv->kv', kc, vc), rtol=1e-10, atol=1e-11)
    idx = pw.select_blocks(qc, kc, 16 ** -0.5, 0.5)
    assert idx.shape == (4, 2)
    score = torch.from_numpy(qc @ (kc * 16 ** -0.5).T)
    assert (np.sort(idx, -1) == np.sort(torch.topk(score, 2, dim=-1).indices.numpy(), -1)).all()


@pytest.mark.parametrize("p", [1, 2])
def test_piecewise_selection_with_bias_ranks_score_plus_log_norm(p):
    """kernel.py:172-174,314-318: with use_bias the ranking is torch.topk of softmax(score + log(norm + 1e-5)).
    The softmax is monotone per row, so the selected set must be topk(score + log(norm + 1e-5)), with the
    norms from torch.norm(p=...) of the flattened chunk matrices: evaluated here with torch on the
    softmax itself, as the reference's wrapper does."""
    q, k, v = _pw_inputs(T=64 * 11 + 5, seed=9)
    qc, kc, vc, hc, H, lens = pw.chunk_reduce(q, k, v, 64)
    NT = qc.shape[0]
    scale = 16 ** -0.5
    idx = pw.select_blocks(qc, kc, scale, 0.3, hc=hc, use_bias=True, p=p)
    top_k = max(1, int(0.3 * NT))
    assert idx.shape == (NT, top_k)
    h_norm = torch.norm(torch.from_numpy(hc).flatten(-2, -1), p=p, dim=-1)
    score = torch.from_numpy(qc) @ (torch.from_numpy(kc) * scale).T + torch.log(h_norm + 1e-5)[None, :]
    want = torch.topk(torch.softmax(score, dim=-1), top_k, dim=-1).indices.numpy()
    assert (np.sort(idx, -1) == np.sort(want, -1)).all()
    # and the bias changes the selection (otherwise the check above pins nothing about it)
    plain = pw.select_blocks(qc, kc, scale, 0.3)
    assert (np.sort(idx, -1) != np.sort(plain, -1)).any()


def test_piecewise_first_order_term_is_taylor_expansion():
    # Small scores: exp(s_ij) ~ exp(sb_ic)(1 + s_ij - sb_ic); the first-order term must
    # move the result towards exact attention (a sanity check; the coefficient itself
    # is pinned by the three tests below).
    q, k, v = _pw_inputs(T=512, K=8, V=4, seed=9)
    q, k = 0.3 * q, 0.3 * k
    NT = 8
    idx = np.stack([np.array([t]) for t in range(NT)])
    ref = torch.nn.functional.scaled_dot_product_attention(
        torch.from_numpy(q)[None], torch.from_numpy(k)[None], torch.from_numpy(v)[None])[0].numpy()
    e0 = np.abs(pw.piecewise_forward(q, k, v, idx, 64, first_order=False) - ref).mean()
    e1 = np.abs(pw.piecewise_forward(q, k, v, idx, 64, first_order=True) - ref).mean()
    assert e1 < 0.5 * e0


def _pw_ragged_case(T, K, V, block, n_sel, seed, scale=None):
    q, k, v = _pw_inputs(T=T, K=K, V=V, seed=seed)
    NT = -(-T // block)
    rng = np.random.default_rng(seed)
    idx = np.stack([rng.permutation(NT)[:n_sel] for _ in range(NT)])
    return q, k, v, idx


# The per-token C evaluation (oracle/piecewise_tokens.c) follows the reference kernel
# step by step in base 2 with the kernel's 9-digit log2(e); the dense numpy closed form
# uses exp().  The constants differ by 6e-10 relative, which for |score| < 20 bounds the
# disagreement of the two by ~2e-8; every coefficient mistake below is 1e-3 or more.
_PW_TOL = 2e-8


@pytest.mark.parametrize("T,K,V,block,n_sel,scale", [
    (200, 16, 8, 64, 1, None),      # ragged last chunk (8 tokens), default scale
    (333, 24, 12, 32, 3, 0.37),     # other block size, explicit scale != K^-0.5
    (129, 8, 16, 64, 2, None),      # last chunk of one token
    (64, 8, 4, 16, 4, 0.5),         # every chunk selected: phases 2 and 3 vanish
])
def test_piecewise_closed_form_matches_per_token_c_evaluation(T, K, V, block, n_sel, scale):
    q, k, v, idx = _pw_ragged_case(T, K, V, block, n_sel, seed=T)
    o_np = pw.piecewise_forward(q, k, v, idx, block, scale=scale)
    o_c = pisa_tokens(q, k, v, idx, block, scale=scale)
    assert np.abs(o_np - o_c).max() <= _PW_TOL * np.abs(o_c).max()


def test_piecewise_coefficient_mistakes_are_caught():
    # The first-order term is additive in the numerator, so a closed form with the term
    # multiplied by f is  o_0 + f (o_1 - o_0).  Each plausible mistake must be far outside
    # the tolerance with which the correct closed form matches the per-token evaluation.
    T, K, V, block, n_sel, scale = 333, 24, 12, 32, 3, 0.37
    q, k, v, idx = _pw_ragged_case(T, K, V, block, n_sel, seed=T)
    o_c = pisa_tokens(q, k, v, idx, block, scale=scale)
    o1 = pw.piecewise_forward(q, k, v, idx, block, scale=scale)
    o0 = pw.piecewise_forward(q, k, v, idx, block, scale=scale, first_order=False)
    tol = _PW_TOL * np.abs(o_c).max()
    assert np.abs(o1 - o_c).max() <= tol
    mistakes = {
        "G/(T - selected tokens)": T / (T - n_sel * block),
        "scale dropped": 1.0 / scale,
        "x0.7": 0.7,
        "sign": -1.0,
        "term missing": 0.0,
        "G/NT instead of G/T": T / (-(-T // block)),
    }
    for name, f in mistakes.items():
        err = np.abs(o0 + f * (o1 - o0) - o_c).max()
        assert err > 1e4 * tol, (name, err, tol)


def test_piecewise_zero_mean_chunks_isolate_first_order_coefficient():
    # Keys centred inside every chunk: all chunk means are 0, every mean score is 0,
    # H = K^T V, and G_i = (number of unselected tokens), independent of q.  Then
    #   o_i = [ sum_{j sel} e^{s_ij} v_j + sum_{j unsel} v_j
    #           + (N_unsel/T) scale sum_{all j} (q_i.k_j) v_j ] / [ sum_{j sel} e^{s_ij} + N_unsel ]
    # evaluated here token by token as (q K^T) V - a different contraction order from the
    # oracle's q (K^T V) - and without any running maximum.
    T, K, V, block, scale = 200, 8, 4, 64, 0.41
    q, k, v = _pw_inputs(T=T, K=K, V=V, seed=21)
    for lo in range(0, T, block):
        k[lo:lo + block] -= k[lo:lo + block].mean(0, keepdims=True)
    idx = np.array([[1], [3], [0], [2]])
    o = pw.piecewise_forward(q, k, v, idx, block, scale=scale)
    s = scale * (q @ k.T)                          # [T,T] exact scores
    lin = (q @ k.T) @ v                            # sum_j (q_i.k_j) v_j
    for t in range(4):
        rows = slice(t * block, min(T, (t + 1) * block))
        sel = np.zeros(T, dtype=bool)
        sel[idx[t, 0] * block:(idx[t, 0] + 1) * block] = True
        n_unsel = float((~sel).sum())
        num = np.exp(s[rows][:, sel]) @ v[sel] + v[~sel].sum(0) + (n_unsel / T) * scale * lin[rows]
        den = np.exp(s[rows][:, sel]).sum(-1) + n_unsel
        np.testing.assert_allclose(o[rows], num / den[:, None], rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(pisa_tokens(q, k, v, idx, block, scale=scale), o, rtol=1e-7, atol=1e-9)
