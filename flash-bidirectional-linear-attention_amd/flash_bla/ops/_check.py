"""Argument validation shared by the dense operators."""
import torch


def check_dense(name, q, k, v, extra=()):
    """The reference's dense wrappers validate nothing (linear_attn/fused.py:456-480);
    the HIP kernels index raw memory, so shapes, dtypes and devices are checked here."""
    tensors = (q, k, v) + tuple(extra)
    for t in tensors:
        if not isinstance(t, torch.Tensor) or t.ndim != 4:
            raise ValueError(f"{name}: tensors must have shape (B, H, L, D)")
    if extra:
        # decoupled operator: q_rope shaped like q, k_rope like k (which, like v, may have another
        # number of tokens than q)
        q_rope, k_rope = extra
        if q_rope.shape != q.shape or k_rope.shape != k.shape:
            raise ValueError(f"{name}: q_rope must be shaped like q and k_rope like k, "
                             f"got {[tuple(t.shape) for t in (q, k) + tuple(extra)]}")
    if q.shape[:2] != k.shape[:2] or q.shape[-1] != k.shape[-1]:
        # k and v may be shorter or longer than q (the PVT-style blocks reduce the keys spatially;
        # the reference reads one length from q, linear_attn/fused.py:355, and runs out of bounds)
        raise ValueError(f"{name}: q and k must agree in batch, head and feature dimensions, "
                         f"got {tuple(q.shape)} and {tuple(k.shape)}")
    if k.shape[:3] != v.shape[:3]:
        raise ValueError(f"{name}: k and v must have matching batch, head and token dimensions")
    if any(t.device != q.device for t in tensors):
        raise ValueError(f"{name}: all tensors must be on the same device")
    if any(t.dtype != q.dtype for t in tensors):
        raise ValueError(f"{name}: all tensors must have the same dtype")
    if not q.is_cuda:
        raise ValueError(f"{name}: tensors must be GPU tensors")
    if q.dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError(f"{name}: dtype must be float16, bfloat16, or float32")
    if not (0 < q.shape[-1] <= 128 and 0 < v.shape[-1] <= 128):
        raise ValueError(f"{name}: key_dim and value_dim must be between 1 and 128")
