"""LinFusion's generalized linear attention block (counterpart of
flash_bla/layers/linfusion.py:26-113) without the diffusers dependency.

The reference subclasses `diffusers.models.attention_processor.Attention`; only the
members that class contributes to this forward are reproduced, under the same
names so that state dicts line up: bias-free `to_q/to_k/to_v`, `to_out =
[Linear(bias), Dropout]`, `heads`, and the head split / merge.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from flash_bla.layers._common import check_mode, torch_linear_attention
from flash_bla.ops.linear_attn.fused import linear_attention
from flash_bla.ops.linear_attn.varlen import varlen_linear_attention


_CU_CACHE = {}


def _equal_cu_seqlens(batch, tokens, device):
    """int32 [0, n, 2n, ...] on `device`, cached per (batch, tokens, device)."""
    key = (batch, tokens, str(device))
    cu = _CU_CACHE.get(key)
    if cu is None:
        cu = torch.arange(0, (batch + 1) * tokens, tokens, dtype=torch.int32, device=device)
        _CU_CACHE[key] = cu
    return cu


def get_none_linear_projection(query_dim, mid_dim=None):
    """Residual feature projection in front of to_q / to_k (linfusion.py:26-38):
    Linear -> LayerNorm -> LeakyReLU -> Linear; identity when mid_dim == -1."""
    if mid_dim == -1:
        return nn.Identity()
    width = mid_dim or query_dim
    return nn.Sequential(nn.Linear(query_dim, width), nn.LayerNorm(width), nn.LeakyReLU(inplace=True),
                         nn.Linear(width, query_dim))


class GeneralizedLinearAttention(nn.Module):
    def __init__(self, query_dim, heads=8, dim_head=64, dropout=0.0, bias=False, out_bias=True,
                 out_dim=None, projection_mid_dim=None):
        super().__init__()
        inner = out_dim if out_dim is not None else dim_head * heads
        self.heads = out_dim // dim_head if out_dim is not None else heads
        self.to_q = nn.Linear(query_dim, inner, bias=bias)
        self.to_k = nn.Linear(query_dim, inner, bias=bias)
        self.to_v = nn.Linear(query_dim, inner, bias=bias)
        self.to_out = nn.ModuleList([nn.Linear(inner, out_dim or query_dim, bias=out_bias), nn.Dropout(dropout)])
        self.add_non_linear_model(projection_mid_dim)

    def add_non_linear_model(self, mid_dim=None):
        query_dim = self.to_q.weight.shape[0]
        self.to_q_ = get_none_linear_projection(query_dim, mid_dim)
        self.to_k_ = get_none_linear_projection(query_dim, mid_dim)

    def head_to_batch_dim(self, x):
        b, n, c = x.shape
        return x.view(b, n, self.heads, c // self.heads).transpose(1, 2).reshape(b * self.heads, n, -1)

    def batch_to_head_dim(self, x):
        bh, n, d = x.shape
        return x.view(bh // self.heads, self.heads, n, d).transpose(1, 2).reshape(bh // self.heads, n, -1)

    def forward(self, hidden_states, encoder_hidden_states=None, attention_mask=None, mode='triton', **kwargs):
        fast = check_mode(mode)
        context = hidden_states if encoder_hidden_states is None else encoder_hidden_states
        q = self.to_q(hidden_states + self.to_q_(hidden_states))
        k = self.to_k(context + self.to_k_(context))
        v = self.to_v(context)
        if fast and q.shape[1] == k.shape[1]:
            # The projections come out token-major, (batch, tokens, heads * dim): that is the
            # packed layout of the variable-length operator with equal lengths, so the head
            # split / merge copies of the reference (linfusion.py:98,102) are not needed at all.
            # The feature map is the operator's: an inference forward of 64-wide heads applies it
            # while loading q and k, anything else maps them first (one launch for both).
            b, n, _ = q.shape
            packed = [t.reshape(b * n, self.heads, -1) for t in (q, k, v)]
            out = varlen_linear_attention(*packed, _equal_cu_seqlens(b, n, q.device), n, eps=1e-4,
                                          feature_map="elu+1")
            return self.to_out[1](self.to_out[0](out.reshape(b, n, -1)))
        q, k, v = (self.head_to_batch_dim(t) for t in (q, k, v))
        if fast:
            b = hidden_states.shape[0]
            q4, k4, v4 = (t.view(b, self.heads, *t.shape[1:]) for t in (q, k, v))
            out = linear_attention(q4, k4, v4, eps=1e-4, feature_map="elu+1").flatten(0, 1)
        else:
            q, k = F.elu(q) + 1.0, F.elu(k) + 1.0
            out = torch_linear_attention(q, k, v, eps=1e-4)
        out = self.batch_to_head_dim(out)
        return self.to_out[1](self.to_out[0](out))
