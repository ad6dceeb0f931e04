"""FLatten focused linear attention (counterpart of flash_bla/layers/focused_la.py:13-96)."""
import torch
import torch.nn as nn
import torch.nn.functional as F

from flash_bla.layers._common import check_mode, merge_heads, split_heads, torch_linear_attention
from flash_bla.layers._pvt import PvtLinearAttentionBase
from flash_bla.ops.linear_attn.fused import linear_attention


class FocusedLinearAttention(PvtLinearAttentionBase):
    def __init__(self, dim, num_patches, num_heads=8, qkv_bias=False, qk_scale=None, attn_drop=0., proj_drop=0.,
                 sr_ratio=1, focusing_factor=3, kernel_size=5):
        super().__init__()
        self._init_common(dim, num_patches, num_heads, qkv_bias, attn_drop, proj_drop, sr_ratio, kernel_size)
        self.q = nn.Linear(dim, dim, bias=qkv_bias)
        self.focusing_factor = focusing_factor

    def _focus(self, t, scale):
        """relu features sharpened by an element-wise power at constant norm."""
        t = (F.relu(t) + 1e-6) / scale
        norm = t.norm(dim=-1, keepdim=True)
        t = t ** self.focusing_factor
        return t / t.norm(dim=-1, keepdim=True) * norm

    def forward(self, x, H, W, mode='triton'):
        fast = check_mode(mode)
        N = x.shape[1]
        k, v = self._keys_values(x, H, W)
        scale = F.softplus(self.scale)
        q, k = self._focus(self.q(x), scale), self._focus(k, scale)
        q, k, v = (split_heads(t, self.num_heads) for t in (q, k, v))
        out = linear_attention(q, k, v) if fast else torch_linear_attention(q, k, v)
        out = merge_heads(out) + self._value_conv(v, N, H, W)
        return self.proj_drop(self.proj(out))
