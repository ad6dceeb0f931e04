"""GPU parity of the piecewise (PISA) operators against the float64 oracle
(oracle/piecewise.py, the closed form) and against oracle/piecewise_tokens.c (a per-token
evaluation that follows the reference kernel's phases with one group).  The reference has
neither a naive implementation nor a test for this operator; the two oracles pin each other
(tests/test_oracle.py) and what is checked here is the mathematics the kernel text defines."""
import numpy as np
import pytest
import torch

from helpers import TOL, assert_parity, max_rel_err, np64
from oracle import piecewise as pw

pytestmark = pytest.mark.gpu


def _inputs(B, H, T, K, V, dtype, seed=0, qk_scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (qk_scale * torch.randn(B, H, T, K, generator=g)).to(dtype)
    k = (qk_scale * torch.randn(B, H, T, K, generator=g)).to(dtype)
    v = torch.randn(B, H, T, V, generator=g).to(dtype)
    return q, k, v


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=str)
@pytest.mark.parametrize("T,K,V,chunk", [(200, 64, 64, 64), (1000, 128, 128, 64), (130, 32, 16, 32),
                                         (257, 64, 128, 64)])
def test_fused_chunk_reduce(dtype, T, K, V, chunk):
    from flash_bla.ops.piecewise_attn.kernel import chunk_reduce_fp32, fused_chunk_reduce
    q, k, v = _inputs(1, 3, T, K, V, dtype, seed=1)
    qc, kc, vc, h, bias = chunk_reduce_fp32(q.cuda(), k.cuda(), v.cuda(), chunk, use_bias=True)
    for hd in range(3):
        rq, rk, rv, rhc, rH, lens = pw.chunk_reduce(np64(q)[0, hd], np64(k)[0, hd], np64(v)[0, hd], chunk)
        assert max_rel_err(qc[0, hd], rq) < 1e-5
        assert max_rel_err(kc[0, hd], rk) < 1e-5
        assert max_rel_err(vc[0, hd], rv) < 1e-5
        assert max_rel_err(h[0, hd], rH) < 2e-5
        ref_norm = np.sqrt((rhc.reshape(rhc.shape[0], -1) ** 2).sum(-1))
        assert max_rel_err(bias[0, hd, 0], ref_norm) < 2e-5
    # the reference-typed variant returns the input dtype and no bias by default
    out = fused_chunk_reduce(q.cuda(), k.cuda(), v.cuda(), chunk)
    assert out[0].dtype == dtype and out[3].dtype == dtype and out[4] is None
    assert out[3].shape == (1, 3, K, V)


def _oracle(q, k, v, indices, scale=None, block=64):
    B, H = q.shape[:2]
    out = np.zeros(v.shape, dtype=np.float64)
    for b in range(B):
        for h in range(H):
            out[b, h] = pw.piecewise_forward(np64(q)[b, h], np64(k)[b, h], np64(v)[b, h],
                                             indices[b, h].cpu().numpy(), block, scale)
    return out


@pytest.mark.parametrize("T,K,V,block,density,dtype", [
    (200, 16, 8, 32, 0.3, torch.float32),       # small head dims, ragged last block, fp32
    (300, 100, 72, 64, 0.25, torch.float16),    # head dims that are not multiples of 16
    (257, 64, 64, 16, 0.2, torch.bfloat16),     # 16-token blocks (MFMA kernel, four query blocks per query tile)
    (400, 128, 128, 128, 0.5, torch.float16),   # 128-token blocks (MFMA kernel, two key tiles per block)
    (300, 64, 64, 48, 0.3, torch.float16),      # a block size the MFMA kernel does not take
    (333, 24, 40, 50, 0.1, torch.float32),      # nothing a power of two
    (256, 64, 64, 64, 0.25, torch.float32),     # the MFMA shape in fp32
    (70, 8, 4, 1, 0.05, torch.float32),         # one-token blocks
    (260, 32, 16, 64, 0.25, torch.bfloat16),    # 16-bit head dims that the state kernel pads
    (700, 96, 80, 64, 0.25, torch.bfloat16),    # 16-bit, 64-token blocks: widened to 128 x 128 for the MFMA kernel
    (130, 8, 120, 64, 0.4, torch.float16),      # widened to 64 x 128
])
def test_shape_generic_kernel_matches_oracle_and_per_token_evaluation(T, K, V, block, density, dtype):
    """Head dims, block sizes and the dtype outside the MFMA kernel's domain run on the
    shape-generic kernel (16-bit inputs with blocks of 16, 32 or a multiple of 64 tokens: on the MFMA kernel,
    head dims other than 64 / 128 through copies widened with zeros): against the float64 closed form and, independently, against the
    per-token C evaluation that follows the reference kernel's phases."""
    from flash_bla.ops.piecewise_attn.kernel import (chunk_reduce_fp32, piecewise_sparse_attention,
                                                     select_blocks)
    from oracle.piecewise_tokens import pisa_tokens
    q, k, v = _inputs(1, 2, T, K, V, dtype, seed=T + K)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    scale = 0.8 * K ** -0.5
    qc, kc, vc, h, _ = chunk_reduce_fp32(qd, kd, vd, block)
    for hd in range(2):
        rq, rk, rv, _, rH, _ = pw.chunk_reduce(np64(q)[0, hd], np64(k)[0, hd], np64(v)[0, hd], block)
        assert max_rel_err(qc[0, hd], rq) < 1e-5 and max_rel_err(kc[0, hd], rk) < 1e-5
        # H = K^T V - sum_c kc_c vc_c^T cancels (to zero for one-token blocks): the scale is K^T V's
        assert max_rel_err(vc[0, hd], rv) < 1e-5 and max_rel_err(h[0, hd], rH, np64(k)[0, hd].T @ np64(v)[0, hd]) < 2e-5
    indices = select_blocks(qc, kc, scale, density)
    NT = -(-T // block)
    assert indices.shape == (1, 2, NT, max(1, int(density * NT)))
    o = piecewise_sparse_attention(qd, kd, vd, density=density, block_size=block, scale=scale, indices=indices)
    assert o.dtype == dtype and o.shape == v.shape
    ref = _oracle(q, k, v, indices, scale=scale, block=block)
    floor = _oracle(q, k, v.abs(), indices, scale=scale, block=block)
    assert_parity(o, ref, dtype, f"T{T} K{K} V{V} block{block}", floor)
    for hd in range(2):
        tok = pisa_tokens(np64(q)[0, hd], np64(k)[0, hd], np64(v)[0, hd], indices[0, hd].cpu().numpy(), block, scale)
        assert_parity(o[0, hd], tok, dtype, f"per-token evaluation, head {hd}", floor[0, hd])
    o2 = piecewise_sparse_attention(qd, kd, vd, density=density, block_size=block, scale=scale)
    assert torch.equal(o, o2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("T,K,V,density", [
    (256, 64, 64, 0.5),
    (200, 64, 64, 0.3),        # ragged last block
    (1000, 128, 128, 0.25),    # BASELINE config 5 head dims
    (640, 128, 64, 0.1),
    (520, 64, 128, 0.4),
])
def test_piecewise_attention_matches_oracle(dtype, T, K, V, density):
    from flash_bla.ops.piecewise_attn.kernel import (chunk_reduce_fp32, piecewise_sparse_attention,
                                                     select_blocks)
    q, k, v = _inputs(1, 2, T, K, V, dtype, seed=2)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    qc, kc, vc, h, _ = chunk_reduce_fp32(qd, kd, vd, 64)
    indices = select_blocks(qc, kc, K ** -0.5, density)
    o = piecewise_sparse_attention(qd, kd, vd, density=density, indices=indices)
    assert o.dtype == dtype and o.shape == v.shape
    ref = _oracle(q, k, v, indices)
    assert_parity(o, ref, dtype, f"T{T} K{K} V{V}")
    # independently of the closed form: the per-token C evaluation of the reference kernel's phases
    from oracle.piecewise_tokens import pisa_tokens
    tok = pisa_tokens(np64(q)[0, 0], np64(k)[0, 0], np64(v)[0, 0], indices[0, 0].cpu().numpy(), 64)
    assert_parity(o[0, 0], tok, dtype, f"per-token evaluation T{T} K{K} V{V}")
    # and with its own selection (same code path as select_blocks)
    o2 = piecewise_sparse_attention(qd, kd, vd, density=density)
    assert torch.equal(o, o2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("high", [(0, 1, 2, 3), (4, 5, 6, 7), (12, 13, 14, 15, 28), (33,)])
def test_row_maximum_sees_every_key_of_a_block(dtype, high):
    """Scores that differ by more than the exponent range of fp32 between groups of keys: keys
    whose index inside their block of 64 is in `high` score +112 (natural units), all others
    -112.  A running maximum that missed a group of keys of a block (one half-wave's keys, one
    register's key) would overflow exp2 and return inf / nan; with the true maximum the
    output is softmax attention over the high keys only."""
    from flash_bla.ops.piecewise_attn.kernel import piecewise_sparse_attention
    T, K, V = 192, 64, 64
    g = torch.Generator().manual_seed(11)
    q = torch.zeros(1, 1, T, K)
    q[..., 0] = 30.0
    k = 0.01 * torch.randn(1, 1, T, K, generator=g)
    k[..., 0] = -30.0
    for j in high:
        k[0, 0, j::64, 0] = 30.0
    v = torch.randn(1, 1, T, V, generator=g)
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    o = piecewise_sparse_attention(q.cuda(), k.cuda(), v.cuda(), density=1.0)
    assert torch.isfinite(o).all()
    ref = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double())
    assert_parity(o, ref, dtype, f"high keys {high}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_all_blocks_selected_is_softmax_attention(dtype):
    from flash_bla.ops.piecewise_attn.kernel import piecewise_sparse_attention
    q, k, v = _inputs(2, 2, 300, 64, 64, dtype, seed=3)
    o = piecewise_sparse_attention(q.cuda(), k.cuda(), v.cuda(), density=1.0)
    ref = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double())
    assert_parity(o, ref, dtype, "density 1")


def test_many_small_blocks_need_more_than_64k_of_lds():
    """2048 blocks of 16 tokens, all selected: four bitmaps and a list of 2048 key tiles next to the tile ring
    take more LDS than a kernel gets by default (the launch raises its limit).  With every block selected
    the result is softmax attention, evaluated here by torch in fp32 on the GPU."""
    from flash_bla.ops.piecewise_attn.kernel import piecewise_sparse_attention
    dtype = torch.float16
    q, k, v = (t.cuda() for t in _inputs(1, 1, 32768, 64, 64, dtype, seed=9, qk_scale=0.5))
    o = piecewise_sparse_attention(q, k, v, density=1.0, block_size=16)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert_parity(o, ref.double().cpu(), dtype, "2048 blocks of 16 tokens, density 1")


def test_small_scores_first_order_branch():
    """Small logits: the linear branch carries real weight and the first-order term matters."""
    from flash_bla.ops.piecewise_attn.kernel import chunk_reduce_fp32, piecewise_sparse_attention
    q, k, v = _inputs(1, 2, 768, 64, 64, torch.float16, seed=4, qk_scale=0.3)
    NT = 12
    indices = torch.arange(NT).view(1, 1, NT, 1).expand(1, 2, NT, 1).contiguous().cuda()
    o = piecewise_sparse_attention(q.cuda(), k.cuda(), v.cuda(), indices=indices, scale=0.5)
    ref = _oracle(q, k, v, indices, scale=0.5)
    assert_parity(o, ref, torch.float16, "first order")


def test_use_bias_selection_and_errors():
    from flash_bla.ops.piecewise_attn.kernel import piecewise_sparse_attention
    q, k, v = _inputs(1, 2, 512, 64, 64, torch.bfloat16, seed=5)
    o = piecewise_sparse_attention(q.cuda(), k.cuda(), v.cuda(), density=0.25, use_bias=True)
    assert torch.isfinite(o).all()
    with pytest.raises(ValueError):
        piecewise_sparse_attention(q.cuda(), k.cuda(), v.cuda(), block_size=0)
    with pytest.raises(ValueError):
        piecewise_sparse_attention(q, k, v)
    big = torch.zeros(1, 1, 8, 192, dtype=torch.float16, device="cuda")  # head dim above 128
    with pytest.raises(NotImplementedError):
        piecewise_sparse_attention(big, big, big)


@pytest.mark.parametrize("dtype,T,K,V,block", [(torch.bfloat16, 1024, 64, 64, 64), (torch.float16, 1500, 128, 128, 64),
                                               (torch.float32, 700, 48, 40, 32)])
def test_use_bias_end_to_end(dtype, T, K, V, block):
    """use_bias=True through the wrapper: the block norms reach the selection (softmax is monotone, so
    the ranking is that of score + log(norm + 1e-5), kernel.py:172-174,314-318) and the attention runs
    on that selection."""
    from flash_bla.ops.piecewise_attn.kernel import (chunk_reduce, chunk_reduce_fp32, piecewise_sparse_attention,
                                                     select_blocks)
    q, k, v = _inputs(1, 2, T, K, V, dtype, seed=21)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    scale, density = K ** -0.5, 0.25
    o = piecewise_sparse_attention(qd, kd, vd, density=density, block_size=block, use_bias=True)
    qc, kc, vc, h, bias = chunk_reduce_fp32(qd, kd, vd, block, True)
    NT = qc.shape[-2]
    assert bias.shape == (1, 2, 1, NT)
    idx = select_blocks(qc, kc, scale, density, bias)
    # the wrapper ran on exactly this selection (with use_bias the statistics come from the kernels that
    # also write the norms, so the comparison keeps the flag)
    assert torch.equal(o, piecewise_sparse_attention(qd, kd, vd, block_size=block, use_bias=True, indices=idx))
    for hd in range(2):
        rq, rk, rv, rhc, _, _ = pw.chunk_reduce(np64(q)[0, hd], np64(k)[0, hd], np64(v)[0, hd], block)
        # the norms the selection saw
        want_norm = np.linalg.norm(rhc.reshape(NT, -1), axis=-1)
        assert max_rel_err(bias[0, hd, 0], want_norm) < 1e-4
        # the selection against the oracle's, as sets; near ties may differ
        want = np.sort(pw.select_blocks(rq, rk, scale, density, hc=rhc, use_bias=True), axis=-1)
        got = idx[0, hd].cpu().numpy()
        differ = (want != got).any(-1)
        assert differ.sum() <= max(1, NT // 20), f"{differ.sum()} of {NT} query blocks select differently"
        # the output on the kernel's own selection against the dense oracle
        ref = pw.piecewise_forward(np64(q)[0, hd], np64(k)[0, hd], np64(v)[0, hd], got, block, scale)
        assert_parity(o[0, hd], ref, dtype, f"use_bias head {hd}")
    # the three-output form of the statistics
    c3 = chunk_reduce(qd, kd, vd, block)
    assert [t.dtype for t in c3] == [dtype] * 3
    assert torch.equal(c3[1], kc.to(dtype)) and torch.equal(c3[2], vc.to(dtype))


@pytest.mark.parametrize("NT,K,top_density", [(256, 128, 0.25), (37, 64, 0.3), (1, 64, 1.0), (130, 128, 0.01),
                                              (64, 64, 1.0)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_block_selection_matches_topk(NT, K, top_density, with_bias):
    """The selection kernel against torch.topk on the same fp32 scores, as sets (torch orders
    by score, the kernel by block index); random scores have no ties."""
    from flash_bla.ops.piecewise_attn.kernel import select_blocks
    g = torch.Generator().manual_seed(NT * 7 + K)
    qc = torch.randn(2, 3, NT, K, generator=g).cuda()
    kc = torch.randn(2, 3, NT, K, generator=g).cuda()
    bias = (torch.rand(2, 3, NT, generator=g) * 4 + 0.1).cuda() if with_bias else None
    scale = K ** -0.5
    idx = select_blocks(qc, kc, scale, top_density, bias)
    top_k = max(1, int(top_density * NT))
    assert idx.dtype == torch.int32 and idx.shape == (2, 3, NT, top_k)
    score = torch.einsum('bhid,bhjd->bhij', qc.double(), kc.double() * scale)
    if with_bias:
        score = score + torch.log(bias.double() + 1e-5).unsqueeze(-2)
    want = torch.topk(score, k=top_k, dim=-1).indices.sort(dim=-1).values
    got = idx.long()
    assert (got[..., 1:] > got[..., :-1]).all(), "indices must be strictly ascending"
    mismatch = (got != want).any(dim=-1)
    if mismatch.any():  # fp32 vs fp64 scores may swap two blocks whose scores agree to ~1e-6
        kth = torch.topk(score, k=min(top_k + 1, NT), dim=-1).values
        gap = (kth[..., top_k - 1] - kth[..., -1]).abs() if top_k < NT else torch.ones_like(kth[..., 0])
        assert (gap[mismatch] < 1e-4).all()


def test_block_selection_ties_go_to_lower_index():
    from flash_bla.ops.piecewise_attn.kernel import select_blocks
    NT, K = 96, 64
    qc = torch.ones(1, 1, NT, K).cuda()
    kc = torch.zeros(1, 1, NT, K)
    kc[0, 0, 10] = 1.0   # one clear winner, everything else ties at 0
    idx = select_blocks(qc, kc.cuda(), 1.0, 5 / NT)
    assert idx.shape[-1] == 5
    assert (idx.cpu() == torch.tensor([0, 1, 2, 3, 10], dtype=torch.int32)).all()


@pytest.mark.parametrize("K,V", [(128, 128), (64, 64), (64, 128)])
def test_selection_lengths_around_the_unrolled_stream(K, V):
    """The kernel walks the selected blocks three at a time: every list length from 1 to 8, with the
    ragged last block inside or outside the list, and lists padded with -1 (no block) in the middle
    and at the end give the result of the unpadded list."""
    from flash_bla.ops.piecewise_attn.kernel import piecewise_sparse_attention
    T, dtype = 9 * 64 + 20, torch.bfloat16
    NT = (T + 63) // 64
    q, k, v = _inputs(1, 1, T, K, V, dtype, seed=77)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    rng = np.random.default_rng(5)
    for ns in range(1, 9):
        lists = [rng.permutation(NT)[:ns] for _ in range(NT)]
        first = np.concatenate([[NT - 1], [b for b in rng.permutation(NT - 1)][:ns - 1]])
        lists[0] = first.astype(lists[1].dtype)  # the ragged block first in one list (no duplicates)
        indices = torch.tensor(np.stack(lists), dtype=torch.int32)[None, None].cuda()
        o = piecewise_sparse_attention(qd, kd, vd, indices=indices)
        assert_parity(o, _oracle(q, k, v, indices), dtype, f"{ns} blocks", _oracle(q, k, v.abs(), indices))
        padded = torch.full((1, 1, NT, min(ns + 3, NT)), -1, dtype=torch.int32)  # (at most NT entries)
        padded[..., 0] = indices[..., 0].cpu()
        padded[..., 2:ns + 1] = indices[..., 1:].cpu()  # a hole at position 1, the rest at the end
        o_padded = piecewise_sparse_attention(qd, kd, vd, indices=padded.cuda())
        assert torch.equal(o, o_padded), f"{ns} blocks, padded list"


@pytest.mark.parametrize("T,K,V,block,dtype", [
    (128 * 5 + 16, 128, 128, 128, torch.bfloat16),   # the last block ends inside its first tile
    (128 * 4 + 100, 64, 64, 128, torch.float16),     # ... inside its second tile
    (192 * 3 + 70, 64, 128, 192, torch.bfloat16),    # three tiles per block
    (256 * 3 + 129, 128, 64, 256, torch.float16),    # four tiles per block
    (128 * 6 + 40, 96, 72, 128, torch.bfloat16),     # widened head dims
])
def test_blocks_of_several_tiles(T, K, V, block, dtype):
    """Blocks of a multiple of 64 tokens run on the MFMA kernel as several 64-key tiles per selected block,
    the query tiles of one block sharing its selection: every list length from 1 to 5 in random block
    order (the ragged last block first in one list, so that its empty tiles sit in the middle of the
    stream), against the float64 closed form and the per-token evaluation; a list padded with -1 gives
    the result of the unpadded one."""
    from flash_bla.ops.piecewise_attn.kernel import piecewise_sparse_attention
    from oracle.piecewise_tokens import pisa_tokens
    NT = -(-T // block)
    q, k, v = _inputs(1, 1, T, K, V, dtype, seed=T + block)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    rng = np.random.default_rng(block + K)
    for ns in range(1, min(NT, 5) + 1):
        lists = [rng.permutation(NT)[:ns] for _ in range(NT)]
        lists[0] = np.concatenate([[NT - 1], rng.permutation(NT - 1)[:ns - 1]]).astype(lists[0].dtype)
        indices = torch.tensor(np.stack(lists), dtype=torch.int32)[None, None].cuda()
        o = piecewise_sparse_attention(qd, kd, vd, block_size=block, indices=indices)
        floor = _oracle(q, k, v.abs(), indices, block=block)
        assert_parity(o, _oracle(q, k, v, indices, block=block), dtype, f"block {block}, {ns} selected", floor)
        if ns == 2:
            tok = pisa_tokens(np64(q)[0, 0], np64(k)[0, 0], np64(v)[0, 0], indices[0, 0].cpu().numpy(), block,
                              K ** -0.5)
            assert_parity(o[0, 0], tok, dtype, f"per-token evaluation, block {block}", floor[0, 0])
            padded = torch.full((1, 1, NT, min(ns + 2, NT)), -1, dtype=torch.int32)
            padded[..., 0] = indices[..., 0].cpu()
            padded[..., 2] = indices[..., 1].cpu()
            assert torch.equal(o, piecewise_sparse_attention(qd, kd, vd, block_size=block, indices=padded.cuda()))
    o_auto = piecewise_sparse_attention(qd, kd, vd, density=0.4, block_size=block)
    assert torch.isfinite(o_auto.float()).all()


@pytest.mark.parametrize("T,K,V,block,dtype", [
    (64 * 5 + 40, 128, 128, 32, torch.bfloat16),   # ragged last block (8 of 32 rows), last query tile with one block
    (64 * 4 + 50, 64, 64, 16, torch.float16),      # ragged last block (2 of 16 rows)
    (64 * 3, 64, 128, 32, torch.float16),          # whole tiles
    (64 * 6 + 17, 128, 64, 16, torch.bfloat16),
    (64 * 4 + 33, 96, 72, 32, torch.bfloat16),     # widened head dims
    (20, 64, 64, 16, torch.float16),               # less than one tile
])
def test_blocks_smaller_than_a_tile(T, K, V, block, dtype):
    """Blocks of 16 / 32 tokens run on the MFMA kernel too: a key tile is put together from 64 / block
    selected blocks of one query block, the queries of the tile's other query blocks are masked.  Every list
    length from 1 to 7 in random block order (odd lengths leave a tile partly empty; the ragged last block
    is first in one list), against the float64 closed form and the per-token evaluation; a list padded
    with -1 in the middle is checked against the oracle of the unpadded one."""
    from flash_bla.ops.piecewise_attn.kernel import piecewise_sparse_attention
    from oracle.piecewise_tokens import pisa_tokens
    NT = -(-T // block)
    q, k, v = _inputs(1, 2, T, K, V, dtype, seed=T + block)
    qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
    rng = np.random.default_rng(block + K + T)
    for ns in range(1, min(NT, 7) + 1):
        heads = []
        for hd in range(2):
            lists = [rng.permutation(NT)[:ns] for _ in range(NT)]
            lists[hd] = np.concatenate([[NT - 1], rng.permutation(NT - 1)[:ns - 1]]).astype(lists[0].dtype)
            heads.append(np.stack(lists))
        indices = torch.tensor(np.stack(heads), dtype=torch.int32)[None].cuda()
        o = piecewise_sparse_attention(qd, kd, vd, block_size=block, indices=indices)
        floor = _oracle(q, k, v.abs(), indices, block=block)
        assert_parity(o, _oracle(q, k, v, indices, block=block), dtype, f"block {block}, {ns} selected", floor)
        if ns == 3:
            tok = pisa_tokens(np64(q)[0, 1], np64(k)[0, 1], np64(v)[0, 1], indices[0, 1].cpu().numpy(), block,
                              K ** -0.5)
            assert_parity(o[0, 1], tok, dtype, f"per-token evaluation, block {block}", floor[0, 1])
            padded = torch.full((1, 2, NT, min(ns + 2, NT)), -1, dtype=torch.int32)
            padded[..., 0] = indices[..., 0].cpu()
            padded[..., 2] = indices[..., 1].cpu()
            padded[..., 3] = indices[..., 2].cpu()
            # (the holes change which blocks share a tile, hence the order of the sums: not bit-equal)
            o_padded = piecewise_sparse_attention(qd, kd, vd, block_size=block, indices=padded.cuda())
            assert_parity(o_padded, _oracle(q, k, v, indices, block=block), dtype, f"block {block}, padded list", floor)
    o_auto = piecewise_sparse_attention(qd, kd, vd, density=0.3, block_size=block)
    assert torch.isfinite(o_auto.float()).all()


@pytest.mark.parametrize("seed", range(3))
def test_random_piecewise_cases(seed):
    """Seeded random lengths (ragged last blocks, one block, many blocks), head dims, densities
    and score scales, with the kernel's own selection and with random, unsorted, duplicate-free
    selections, against the float64 oracle; the block statistics without bias are checked too."""
    from flash_bla.ops.piecewise_attn.kernel import chunk_reduce_fp32, piecewise_sparse_attention, select_blocks
    rng = np.random.default_rng(3000 + seed)
    for case in range(5):
        K, V = int(rng.choice([64, 128])), int(rng.choice([64, 128]))
        T = int(rng.choice([1, 63, 64, 65, 200, 511, 640, 1025, 1500]))
        H = int(rng.integers(1, 4))
        dtype = [torch.float16, torch.bfloat16][int(rng.integers(0, 2))]
        density = float(rng.choice([0.05, 0.25, 0.5, 1.0]))
        qk_scale = float(rng.choice([0.3, 1.0]))
        q, k, v = _inputs(1, H, T, K, V, dtype, seed=seed * 10 + case, qk_scale=qk_scale)
        qd, kd, vd = q.cuda(), k.cuda(), v.cuda()
        qc, kc, vc, h, _ = chunk_reduce_fp32(qd, kd, vd, 64)
        for hd in range(H):
            rq, rk, rv, _, rH, _ = pw.chunk_reduce(np64(q)[0, hd], np64(k)[0, hd], np64(v)[0, hd], 64)
            assert max_rel_err(qc[0, hd], rq) < 1e-5 and max_rel_err(kc[0, hd], rk) < 1e-5
            assert max_rel_err(vc[0, hd], rv) < 1e-5 and max_rel_err(h[0, hd], rH) < 2e-5
        NT = (T + 63) // 64
        if case % 2 == 0:
            indices = select_blocks(qc, kc, K ** -0.5, density)
        else:  # an arbitrary selection in arbitrary order
            ns = max(1, int(density * NT))
            indices = torch.stack([torch.stack([torch.tensor(rng.permutation(NT)[:ns]) for _ in range(NT)])
                                   for _ in range(H)])[None].to(torch.int32).cuda()
        o = piecewise_sparse_attention(qd, kd, vd, density=density, indices=indices)
        ref = _oracle(q, k, v, indices)
        # The probabilities enter the value product rounded to 16 bits (as in the reference
        # kernel, kernel.py:231), so the error scales with sum_j p_j |v_j| / sum_j p_j, which for
        # flat attention over zero-mean values is much larger than |o| itself: that weighted
        # mean of |v| (the same oracle on |v|) is the scale floor, like dq_mag for gradients.
        floor = _oracle(q, k, v.abs(), indices)
        assert_parity(o, ref, dtype, f"T{T} K{K} V{V} H{H} density{density} scale{qk_scale} {dtype}", floor)
