"""Piecewise (PISA) sparse attention, forward only (drop-in for
flash_bla/ops/piecewise_attn/kernel.py:152-176,295-333).

Key blocks of `block_size` tokens are ranked per query block by the product of block-mean
queries and keys; the top `density` fraction is attended exactly (softmax), every
other block contributes through its mean key and value sum (zeroth order) plus a
first-order correction with H = sum_c (K_c - kc_c)^T V_c.  All block statistics
are kept in fp32 (the reference stores them in the input dtype).

Deliberate difference from the reference's kernel: the running normaliser of the linear branch is
rescaled together with the running maximum.  The Triton kernel rescales its accumulator and its
exact-branch sum but not that normaliser when the maximum grows between groups of unselected blocks
(kernel.py:263-276), so with more blocks than one group (its autotuned GROUP_SIZE) its output depends
on the group size; with one group both agree.  What is computed here is the group-independent value.

Two kernels: fp16 / bf16 inputs with blocks of 16, 32 or a multiple of 64 tokens run on the MFMA kernel
(head dims other than 64 / 128 through copies widened with zeros inside the library; blocks below 64 at
block / 64 of the exact branch's speed); other block sizes and fp32 inputs run on a shape-generic fp32
kernel (correct, one to two orders of magnitude slower).
"""
import torch

from flash_bla import _hip


def _check(q, k, v):
    for t in (q, k, v):
        if not isinstance(t, torch.Tensor) or t.ndim != 4:
            raise ValueError("q, k, and v must have shape (B, H, T, D)")
    if q.shape != k.shape or q.shape[:3] != v.shape[:3]:
        raise ValueError(f"mismatching shapes: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    if not (q.dtype == k.dtype == v.dtype) or not (q.device == k.device == v.device):
        raise ValueError("q, k, and v must have the same dtype and device")
    if not q.is_cuda:
        raise ValueError("piecewise attention needs GPU tensors")


def fused_chunk_reduce(q, k, v, chunk_size, use_bias=False, p=2):
    """Block statistics (kernel.py:152-176): qc, kc = chunk means `(B,H,N,K)`, vc = chunk
    sums `(B,H,N,V)`, h = sum over chunks of `(K_c - kc_c)^T V_c` `(B,H,K,V)` and, with
    `use_bias`, the p-norm of every chunk's matrix as `(B,H,1,N)` (else None).
    Returned in the input dtype like the reference; `chunk_reduce_fp32` keeps fp32."""
    qc, kc, vc, h, bias = chunk_reduce_fp32(q, k, v, chunk_size, use_bias, p)
    return qc.to(k.dtype), kc.to(k.dtype), vc.to(v.dtype), h.to(v.dtype), bias


def chunk_reduce(q, k, v, chunk_size):
    """The block means and value sums alone (kernel.py:131-149): qc, kc `(B,H,N,K)`, vc `(B,H,N,V)`
    in the input dtype."""
    qc, kc, vc, _, _ = chunk_reduce_fp32(q, k, v, chunk_size)
    return qc.to(k.dtype), kc.to(k.dtype), vc.to(v.dtype)


def chunk_reduce_fp32(q, k, v, chunk_size, use_bias=False, p=2):
    _check(q, k, v)
    qc, kc, vc, h, h_norm = _hip.chunk_reduce(q.contiguous(), k.contiguous(), v.contiguous(),
                                              int(chunk_size), use_bias, p)
    return qc, kc, vc, h, (h_norm[..., None, :] if use_bias else None)


def select_blocks(qc, kc, scale, density, bias=None):
    """Top-k key blocks per query block (kernel.py:304-318): int32 indices `(B,H,N,top_k)` in
    ascending block order (the reference's torch.topk orders them by score; the attention
    result does not depend on the order).  `bias`: optional per-block norms `(B,H,N)`."""
    NT = qc.shape[-2]
    top_k = max(1, int(density * NT))
    qc = qc.float().contiguous()
    kc = kc.float().contiguous()
    if bias is not None:
        bias = bias.float().contiguous()
    return _hip.select_blocks(qc, kc, bias, top_k, scale)


def piecewise_sparse_attention(q, k, v, density=0.1, block_size=64, scale=None, use_bias=False,
                               indices=None):
    """
    Args:
        q, k: `(B, H, T, K)`; v: `(B, H, T, V)`; fp16, bf16 or fp32, K and V up to 128.
        density: fraction of key blocks attended exactly per query block (at least one).
        block_size: tokens per block (the MFMA kernel takes 16, 32 and multiples of 64; other
            sizes take the shape-generic kernel).
        scale: score scale, default `K ** -0.5`.
        use_bias: rank blocks by softmax(score + log(norm of the block's first-order matrix)).
        indices: optional precomputed selection `(B, H, N, top_k)` (not in the reference;
            used to share a selection between implementations).
    Returns `(B, H, T, V)` in the input dtype.  Forward only, as in the reference.
    """
    _check(q, k, v)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    K = k.shape[-1]
    scale = K ** -0.5 if scale is None else scale
    if block_size < 1:
        raise ValueError(f"block_size must be positive, got {block_size}")
    if not _hip.piecewise_supported(q, v, block_size):
        raise NotImplementedError(
            "piecewise_sparse_attention on gfx950 needs fp16/bf16/fp32 inputs, head dims up to 128 and a "
            "number of blocks whose selection flags fit LDS "
            f"(got dtype {q.dtype}, K={K}, V={v.shape[-1]}, block_size={block_size}, T={q.shape[-2]})")
    qc, kc, vc, h, bias = chunk_reduce_fp32(q, k, v, block_size, use_bias)
    if indices is None:
        indices = select_blocks(qc, kc, scale, density, bias)
    indices = indices.to(torch.int32).contiguous()
    return _hip.piecewise_fwd(q, k, v, kc, vc, h, indices, block_size, scale)
