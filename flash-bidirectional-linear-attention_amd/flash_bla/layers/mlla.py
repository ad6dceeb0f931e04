"""Mamba-like linear attention block (counterpart of flash_bla/layers/mlla.py:10-99):
elu+1 features, 2-D rotary numerator features, depth-wise conv positional term."""
import torch
import torch.nn as nn

from flash_bla.layers._common import check_mode, merge_heads, split_heads, torch_linear_attention
from flash_bla.ops.feature_map import elu_plus_one
from flash_bla.ops.linear_attn.decoupled import decoupled_la


class RoPE(nn.Module):
    """Rotary embedding over a grid of channel dims (mlla.py:10-36): the feature dim is
    cut into complex pairs, each rotated by position * base^(-j/k_max) along one grid axis."""

    def __init__(self, shape, base=10000):
        super().__init__()
        *grid, feature_dim = shape
        k_max = feature_dim // (2 * len(grid))
        assert feature_dim % k_max == 0
        freqs = base ** (-torch.arange(k_max) / k_max)
        coords = torch.meshgrid([torch.arange(n) for n in grid], indexing='ij')
        angles = torch.cat([c.unsqueeze(-1) * freqs for c in coords], dim=-1)
        self.register_buffer('rotations', torch.stack([angles.cos(), angles.sin()], dim=-1))

    def forward(self, x):
        pairs = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
        return torch.view_as_real(torch.view_as_complex(self.rotations) * pairs).flatten(-2)


class MambaLikeLinearAttention(nn.Module):
    def __init__(self, dim, input_resolution, num_heads, qkv_bias=True, **kwargs):
        super().__init__()
        self.dim, self.input_resolution, self.num_heads = dim, input_resolution, num_heads
        self.qk = nn.Linear(dim, dim * 2, bias=qkv_bias)
        self.elu = nn.ELU()
        self.lepe = nn.Conv2d(dim, dim, 3, padding=1, groups=dim)
        self.rope = RoPE(shape=(input_resolution[0], input_resolution[1], dim))

    def forward(self, x, mode='triton'):
        fast = check_mode(mode)
        b, n, c = x.shape
        side = int(n ** 0.5)
        qk = self.qk(x)
        if fast:  # one launch over the joint projection
            q, k = elu_plus_one(qk).chunk(2, dim=-1)
        else:
            q, k = (self.elu(t) + 1.0 for t in qk.chunk(2, dim=-1))
        rot = [self.rope(t.reshape(b, side, side, c)).reshape(b, n, c).to(x.dtype) for t in (q, k)]
        q, k, v, q_rope, k_rope = (split_heads(t, self.num_heads) for t in (q, k, x, *rot))
        if fast:
            out = decoupled_la(q, k, q_rope, k_rope, v, scale=n ** -1.0)
        else:
            out = torch_linear_attention(q, k, v, q_num=q_rope, k_num=k_rope)
        grid = merge_heads(v).reshape(b, side, side, c).permute(0, 3, 1, 2)
        return merge_heads(out) + self.lepe(grid).permute(0, 2, 3, 1).reshape(b, n, c)

    def extra_repr(self):
        return f'dim={self.dim}, num_heads={self.num_heads}'
