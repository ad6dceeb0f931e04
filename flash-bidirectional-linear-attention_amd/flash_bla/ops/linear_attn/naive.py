"""Plain-torch formulas of the operators (same names and arguments as
flash_bla/ops/linear_attn/naive.py:6-43).  They run on whatever device their inputs
live on and are what the layers' ``mode='torch'`` uses; the HIP operators never
call them."""
import torch


def _state_attention(q_num, k_num, q_den, k_den, v, scale, eps):
    """One formula for all three operators.  The last two dims are (tokens, features):

        o_t = (q_num_t S) / (q_den_t . mean_t(k_den) + eps),   S = k_num^T (scale v)

    `scale` multiplies v before the contraction so that the state stays in range for
    16-bit inputs."""
    state = k_num.mT @ (v * scale)                          # [..., K, V]
    denom = q_den @ k_den.mean(dim=-2).unsqueeze(-1) + eps  # [..., T, 1]
    return (q_num @ state) / denom


def naive_linear_attn(q, k, v, scale=None):
    return _state_attention(q, k, q, k, v, 1.0 / k.shape[-2] if scale is None else scale, 1e-6)


def naive_decoupled_la(q, k, q_rope, k_rope, v, scale=None):
    return _state_attention(q_rope, k_rope, q, k, v, 1.0 / k.shape[-2] if scale is None else scale, 1e-6)


def naive_varlen_linear_attn(q, k, v, cu_seqlens, scale=None, eps=1e-6):
    """Packed [T, H, D] tensors: every [cu_seqlens[i], cu_seqlens[i+1]) range is one sequence
    with its own state and, when `scale` is None, its own 1 / length."""
    edges = cu_seqlens.tolist()
    pieces = []
    for lo, hi in zip(edges, edges[1:]):
        q_s, k_s, v_s = (x[lo:hi].movedim(0, 1) for x in (q, k, v))  # heads first
        o_s = _state_attention(q_s, k_s, q_s, k_s, v_s, 1.0 / max(hi - lo, 1) if scale is None else scale, eps)
        pieces.append(o_s.movedim(1, 0))
    return torch.cat(pieces, dim=0)
