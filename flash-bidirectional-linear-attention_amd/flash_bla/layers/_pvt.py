"""What the two PVT-style blocks (FLatten focused attention, PolaFormer) share:
optional spatial reduction of the key/value tokens, a learned positional term on
the keys, a depth-wise convolution of the values added to the output."""
import torch
import torch.nn as nn
import torch.nn.functional as F


class PvtLinearAttentionBase(nn.Module):
    def _init_common(self, dim, num_patches, num_heads, qkv_bias, attn_drop, proj_drop, sr_ratio, kernel_size):
        assert dim % num_heads == 0, f"dim {dim} should be divided by num_heads {num_heads}."
        self.dim, self.num_heads, self.sr_ratio = dim, num_heads, sr_ratio
        head_dim = dim // num_heads
        self.kv = nn.Linear(dim, dim * 2, bias=qkv_bias)
        self.attn_drop = nn.Dropout(attn_drop)
        self.proj = nn.Linear(dim, dim)
        self.proj_drop = nn.Dropout(proj_drop)
        if sr_ratio > 1:
            self.sr = nn.Conv2d(dim, dim, kernel_size=sr_ratio, stride=sr_ratio)
            self.norm = nn.LayerNorm(dim)
        self.dwc = nn.Conv2d(head_dim, head_dim, kernel_size, groups=head_dim, padding=kernel_size // 2)
        self.scale = nn.Parameter(torch.zeros(1, 1, dim))
        self.positional_encoding = nn.Parameter(torch.zeros(1, num_patches // (sr_ratio * sr_ratio), dim))
        return head_dim

    def _keys_values(self, x, H, W):
        B, N, C = x.shape
        if self.sr_ratio > 1:
            x = self.norm(self.sr(x.transpose(1, 2).reshape(B, C, H, W)).flatten(2).transpose(1, 2))
        k, v = self.kv(x).chunk(2, dim=-1)
        return k + self.positional_encoding, v

    def _value_conv(self, v, N, H, W):
        """v: (B, heads, n, d) -> depth-wise conv on the H x W grid -> (B, N, C)."""
        B, heads, n, d = v.shape
        if self.sr_ratio > 1:
            v = F.interpolate(v.transpose(-2, -1).reshape(B * heads, d, n), size=N, mode='linear')
            v = v.reshape(B, heads, d, N).transpose(-2, -1)
        v = v.reshape(B * heads, H, W, d).permute(0, 3, 1, 2)
        return self.dwc(v).reshape(B, heads * d, N).transpose(1, 2)
