"""PolaFormer polarity-aware linear attention (counterpart of
flash_bla/layers/polaformer.py:10-108): positive and negative parts of q, k are
kept as separate features, the same-sign and opposite-sign pairings attend to the
two halves of the value channels."""
import torch
import torch.nn as nn
import torch.nn.functional as F

from flash_bla.layers._common import check_mode, merge_heads, split_heads, torch_linear_attention
from flash_bla.layers._pvt import PvtLinearAttentionBase
from flash_bla.ops.linear_attn.paired import paired_linear_attention


class PolaLinearAttention(PvtLinearAttentionBase):
    def __init__(self, dim, num_patches, num_heads=8, qkv_bias=False, qk_scale=None, attn_drop=0., proj_drop=0.,
                 sr_ratio=1, kernel_size=5, alpha=4):
        super().__init__()
        self.head_dim = self._init_common(dim, num_patches, num_heads, qkv_bias, attn_drop, proj_drop, sr_ratio,
                                          kernel_size)
        self.qg = nn.Linear(dim, 2 * dim, bias=qkv_bias)
        self.power = nn.Parameter(torch.zeros(1, num_heads, 1, self.head_dim))
        self.alpha = alpha

    def forward(self, x, H, W, mode='triton'):
        fast = check_mode(mode)
        N = x.shape[1]
        q, gate = self.qg(x).chunk(2, dim=-1)
        k, v = self._keys_values(x, H, W)
        scale = F.softplus(self.scale)
        power = 1 + self.alpha * torch.sigmoid(self.power)
        q, k, v = (split_heads(t, self.num_heads) for t in (q / scale, k / scale, v))
        q_pos, q_neg, k_pos, k_neg = (F.relu(t) ** power for t in (q, -q, k, -k))
        q_same = torch.cat([q_pos, q_neg], dim=-1)
        q_opp = torch.cat([q_neg, q_pos], dim=-1)
        k_both = torch.cat([k_pos, k_neg], dim=-1)
        if fast:  # both pairings on one state pass over the shared keys and values
            out = torch.cat(paired_linear_attention(q_same, q_opp, k_both, v), dim=-1)
        else:
            v_same, v_opp = v.chunk(2, dim=-1)
            out = torch.cat([torch_linear_attention(q_same, k_both, v_same),
                             torch_linear_attention(q_opp, k_both, v_opp)], dim=-1)
        out = (merge_heads(out) + self._value_conv(v, N, H, W)) * gate
        return self.proj_drop(self.proj(out))
