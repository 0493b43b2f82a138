"""Alternative compression networks for `SparseAttention(compress_mlp=...)`: each maps the
windows 'b h w n d' (n = compress_block_size tokens) to one compressed key or value 'b h w d'.
Same class names, constructor arguments and parameter names as
native_sparse_attention_pytorch/compress_networks.py:19-241, so that checkpoints load.

All of them are dense projections: they run as (batched) hipBLASLt GEMMs.  The per-head
networks (compress_networks.py:73-138) are written as one batched GEMM over the head axis
(`torch.bmm` on 'h (b w) i' x 'h i o') instead of a general einsum, which keeps a single
strided-batched launch per layer whatever the head count.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn


class HeadwiseLinear(nn.Module):
    """y[b,h,w,:] = x[b,h,w,:] @ weight[h] (+ bias[h]): every head owns its projection.
    Parameter shapes and initialisation follow the einops mixing layer the reference uses
    (compress_networks.py:87-91): weight 'h i o' ~ U(+-sqrt(3/i)), bias [1,h,1,o] ~ U(+-sqrt(1/i))."""

    def __init__(self, heads: int, dim_in: int, dim_out: int, bias: bool = True):
        super().__init__()
        wb, bb = (3 / dim_in) ** 0.5, (1 / dim_in) ** 0.5
        self.weight = nn.Parameter(torch.zeros(heads, dim_in, dim_out).uniform_(-wb, wb))
        self.bias = nn.Parameter(torch.zeros(1, heads, 1, dim_out).uniform_(-bb, bb)) if bias else None

    def forward(self, x):                                   # 'b h w i -> b h w o'
        b, h, w, i = x.shape
        xh = x.permute(1, 0, 2, 3).reshape(h, b * w, i)
        y = torch.bmm(xh, self.weight.to(xh.dtype))
        if self.bias is not None:
            y = y + self.bias[0].to(xh.dtype)
        return y.reshape(h, b, w, self.weight.shape[-1]).permute(1, 0, 2, 3)


class GroupedMLP(nn.Module):
    """Two-layer MLP per kv head over the flattened window (compress_networks.py:73-101;
    the network train.py:100-104 installs)."""

    def __init__(self, dim_head, compress_window_size, heads, expand_factor=1.):
        super().__init__()
        dim = dim_head * compress_window_size
        hidden = int(dim * expand_factor)
        self.net = nn.Sequential(HeadwiseLinear(heads, dim, hidden), nn.ReLU(), HeadwiseLinear(heads, hidden, dim_head))

    def forward(self, kv):                                  # 'b h w n d -> b h w d'
        return self.net(kv.flatten(-2))


class SingleProjection(nn.Module):
    """One projection (compress_networks.py:105-138): shared across heads over the flattened
    window, or - with heads > 1 - the window's tokens summed and projected per head."""

    def __init__(self, dim_head, compress_window_size, heads=1):
        super().__init__()
        if heads > 1:
            self.compress = HeadwiseLinear(heads, dim_head, dim_head, bias=False)
        else:
            self.compress = nn.Sequential(nn.Flatten(-2), nn.Linear(dim_head * compress_window_size, dim_head, bias=False))
        self.grouped = heads > 1

    def forward(self, kv):
        return self.compress(kv.sum(dim=-2)) if self.grouped else self.compress(kv)


class ConvLinearCompress(nn.Module):
    """Grouped strided convolution, one group per head (compress_networks.py:19-44).  Window w
    of the output sees tokens [w*n, (w+1)*n) of the flattened windows, i.e. exactly window w."""

    def __init__(self, heads, dim_head, compress_window_size):
        super().__init__()
        self.heads = heads
        self.conv = nn.Conv1d(heads * dim_head, heads * dim_head, compress_window_size, stride=compress_window_size, groups=heads)

    def forward(self, kv):
        b, h, w, n, d = kv.shape
        x = kv.permute(0, 1, 4, 2, 3).reshape(b, h * d, w * n)
        if w == 0:
            return kv.new_zeros(b, h, 0, d)
        return self.conv(x).reshape(b, h, d, w).permute(0, 1, 3, 2)


class AttentionPool(nn.Module):
    """Softmax pooling over the window's tokens with learned per-feature logits, initialised to
    the identity (compress_networks.py:48-69)."""

    def __init__(self, dim_head, compress_window_size):
        super().__init__()
        self.to_attn_logits = nn.Linear(dim_head, dim_head, bias=False)
        self.to_attn_logits.weight.data.copy_(torch.eye(dim_head))

    def forward(self, kv):
        return (kv * self.to_attn_logits(kv).softmax(dim=-2)).sum(dim=-2)


class SimpleMultiheadSelfAttention(nn.Module):
    def __init__(self, dim, num_heads, dropout=0.0):
        super().__init__()
        assert dim % num_heads == 0, "Hidden dimension must be divisible by number of heads"
        self.dim, self.num_heads, self.head_dim = dim, num_heads, dim // num_heads
        self.q_proj, self.k_proj, self.v_proj, self.out_proj = (nn.Linear(dim, dim) for _ in range(4))
        self.attn_dropout_p = dropout

    def forward(self, x):
        B, L, D = x.shape
        split = lambda t: t.view(B, L, self.num_heads, self.head_dim).transpose(1, 2)
        o = F.scaled_dot_product_attention(split(self.q_proj(x)), split(self.k_proj(x)), split(self.v_proj(x)),
                                           dropout_p=self.attn_dropout_p if self.training else 0.0)
        return self.out_proj(o.transpose(1, 2).reshape(B, L, D))


class SimpleTransformerFeedForward(nn.Module):
    def __init__(self, dim, hidden_dim, dropout=0.0):
        super().__init__()
        self.fc1, self.fc2 = nn.Linear(dim, hidden_dim), nn.Linear(hidden_dim, dim)
        self.act, self.dropout = nn.GELU(), nn.Dropout(dropout)

    def forward(self, x):
        return self.dropout(self.fc2(self.dropout(self.act(self.fc1(x)))))


class SimpleTransformerLayer(nn.Module):
    def __init__(self, dim, num_heads, ff_hidden_dim=None, dropout=0.0):
        super().__init__()
        self.norm1, self.norm2 = nn.RMSNorm(dim), nn.RMSNorm(dim)
        self.attn = SimpleMultiheadSelfAttention(dim, num_heads, dropout=dropout)
        self.ff = SimpleTransformerFeedForward(dim, ff_hidden_dim or dim * 4, dropout=dropout)

    def forward(self, x):
        x = x + self.attn(self.norm1(x))
        return x + self.ff(self.norm2(x))


class CompressTransformer(nn.Module):
    """Small bidirectional transformer over the tokens of each window ('(b w) n (h d)'); the
    window's compressed vector is its last token after the last layer, whose feed-forward is
    applied to that token only (compress_networks.py:205-241)."""

    def __init__(self, num_layers, dim, num_heads, ff_hidden_dim=None, dropout=0.0):
        super().__init__()
        self.layers = nn.ModuleList([SimpleTransformerLayer(dim, num_heads, ff_hidden_dim, dropout) for _ in range(num_layers)])
        self.num_layers = num_layers

    def forward(self, x):
        b, h, w, n, d = x.shape
        t = x.permute(0, 2, 3, 1, 4).reshape(b * w, n, h * d)
        for layer in self.layers[:-1]:
            t = layer(t)
        last = self.layers[-1]
        t = t + last.attn(last.norm1(t))
        tok = t[:, -1:]
        tok = tok + last.ff(last.norm2(tok))
        return tok.reshape(b, w, h, d).permute(0, 2, 1, 3)
