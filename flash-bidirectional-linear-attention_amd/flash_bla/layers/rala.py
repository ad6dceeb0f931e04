"""RALA block (counterpart of flash_bla/layers/rala.py:8-87): keys reweighted by a
softmax "efficiency" score against the mean query, rotary numerator, output gate."""
import torch
import torch.nn as nn

from flash_bla.layers._common import check_mode, merge_heads, split_heads, torch_linear_attention
from flash_bla.layers.mlla import RoPE
from flash_bla.ops.linear_attn.decoupled import decoupled_la


class RALALinearAttention(nn.Module):
    def __init__(self, dim, input_resolution, num_heads, qkv_bias=True, **kwargs):
        super().__init__()
        self.dim, self.input_resolution, self.num_heads = dim, input_resolution, num_heads
        self.head_dim = dim // num_heads
        self.scale = self.head_dim ** -0.5
        self.qkvo = nn.Linear(dim, dim * 4, bias=qkv_bias)
        self.elu = nn.ELU()
        self.lepe = nn.Conv2d(dim, dim, 5, padding=2, groups=dim)
        self.rope = RoPE(shape=(input_resolution[0], input_resolution[1], self.head_dim))
        self.proj = nn.Linear(dim, dim)

    def forward(self, x, mode='triton'):
        fast = check_mode(mode)
        b, n, c = x.shape
        side = int(n ** 0.5)
        q, k, v, gate = self.qkvo(x).chunk(4, dim=-1)
        lepe = self.lepe(v.reshape(b, side, side, c).permute(0, 3, 1, 2)).permute(0, 2, 3, 1).reshape(b, n, c)
        q, k, v = (split_heads(t, self.num_heads) for t in (self.elu(q) + 1.0, self.elu(k) + 1.0, v))
        # efficiency reweighting: softmax over tokens of scale * mean(q) . k_j, times n
        eff = torch.softmax(self.scale * q.mean(dim=-2, keepdim=True) @ k.transpose(-1, -2), dim=-1)
        k = k * eff.transpose(-1, -2) * n
        grid = (b, self.num_heads, side, side, self.head_dim)
        q_rope = self.rope(q.reshape(grid)).reshape(q.shape).to(x.dtype).contiguous()
        k_rope = self.rope(k.reshape(grid)).reshape(k.shape).to(x.dtype).contiguous()
        if fast:
            out = decoupled_la(q, k.contiguous(), q_rope, k_rope, v, scale=n ** -1.0)
        else:
            out = torch_linear_attention(q, k, v, q_num=q_rope, k_num=k_rope)
        return self.proj((merge_heads(out) + lepe) * gate)

    def extra_repr(self):
        return f'dim={self.dim}, num_heads={self.num_heads}'
