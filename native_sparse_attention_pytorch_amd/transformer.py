"""Decoder-only transformer around `SparseAttention`: the training-forward harness of the
reference (native_sparse_attention_pytorch/transformer.py:130-138 FeedForward, :142-211
construction, :254-330 forward, :213-252 sampling with or without the per-layer caches) with the
same constructor arguments and parameter names."""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch import nn

from .sparse_attention import SparseAttention


def FeedForward(dim, expansion_factor=4.):
    hidden = int(dim * expansion_factor)
    return nn.Sequential(nn.RMSNorm(dim), nn.Linear(dim, hidden), nn.GELU(), nn.Linear(hidden, dim))


class Transformer(nn.Module):
    def __init__(self, num_tokens, dim, depth, dim_head=64, heads=8, kv_heads=None, ff_expansion_factor=4.,
                 use_sparse_attn=True, causal=True, use_flex_sliding_window=False, use_flex_fine_selection=False,
                 use_triton_fine_selection=False, sparse_attn_kwargs: dict | None = None):
        super().__init__()
        if not use_sparse_attn:
            raise NotImplementedError("only the sparse-attention model is provided (the dense baseline is not part of the hot path)")
        # use_flex_sliding_window / use_flex_fine_selection / use_triton_fine_selection choose between the reference's
        # backends for the same masks (transformer.py:154-177, 281-296); accepted so that the reference's training script
        # constructs this model unchanged, and ignored: the HIP kernels always run
        assert not (use_flex_fine_selection and use_triton_fine_selection), 'either using flex or custom triton kernel for fine attn, but not both'
        sparse_attn_kwargs = dict(sparse_attn_kwargs or dict(sliding_window_size=32, compress_block_size=4,
                                                             compress_block_sliding_stride=4, selection_block_size=4,
                                                             num_selected_blocks=4))
        self.token_emb = nn.Embedding(num_tokens, dim)
        self.causal = causal
        layers = []
        for _ in range(depth):
            attn = SparseAttention(dim=dim, dim_head=dim_head, heads=heads, kv_heads=kv_heads, causal=causal,
                                   use_triton_kernel=use_triton_fine_selection, **sparse_attn_kwargs)
            layers.append(nn.ModuleList([attn, FeedForward(dim=dim, expansion_factor=ff_expansion_factor)]))
        self.layers = nn.ModuleList(layers)
        self.norm = nn.RMSNorm(dim)
        self.to_logits = nn.Linear(dim, num_tokens, bias=False)

    @staticmethod
    def _feed_forward(ff, tokens):
        """The feed-forward block (transformer.py:142-152 of the reference: norm, linear, GELU, linear).  While a HIP graph is
        being recorded (training.GraphedStep) the two projections go through ops.linear, whose bias gradients are column sums
        by this library's kernel: the library's own sum records a memset node that replays wrongly on this platform."""
        from . import ops
        if not (ops.capturing() and torch.is_grad_enabled() and tokens.dtype == torch.bfloat16 and isinstance(ff, nn.Sequential) and len(ff) == 4):
            return ff(tokens)
        norm, up, act, down = ff
        plain = SparseAttention._plain
        if not (plain(ff, nn.Sequential) and plain(norm, nn.RMSNorm) and plain(up, nn.Linear) and plain(act, nn.GELU) and plain(down, nn.Linear)):
            return ff(tokens)
        return ops.linear(act(ops.linear(norm(tokens), up.weight, up.bias)), down.weight, down.bias)

    def forward(self, ids, return_loss=False, disable_flex=False, disable_triton_kernel=False, cache=None, return_cache=False):
        if return_loss:
            ids, labels = ids[:, :-1], ids[:, 1:]
        if torch.is_grad_enabled() and ids.is_cuda and not getattr(self, "_recording_warmup", False):
            from . import ops
            if not ops.capturing():
                self._launched_grad_steps = True      # training.GraphedStep must be recorded before the first of these
        # with caches only the newest token is embedded and every layer takes one decode step
        tokens = self.token_emb(ids if cache is None else ids[:, -1:])
        layer_caches = iter(cache or [])
        caches = []
        for attn, ff in self.layers:
            if return_cache or cache is not None:
                attn_out, layer_cache = attn(tokens, cache=next(layer_caches, None), return_cache=True)
            else:
                attn_out, layer_cache = attn(tokens), None
            caches.append(layer_cache)
            tokens = attn_out + tokens
            tokens = self._feed_forward(ff, tokens) + tokens
        logits = self.to_logits(self.norm(tokens))
        if not return_loss:
            return (logits, caches) if return_cache else logits
        # (the mean over all tokens, as transformer.py:330 takes it over 'b l n'; with the classes as the last axis the softmax
        # runs over contiguous rows - the transposed view goes through the strided kernels: 0.32 ms instead of ~10 us a step)
        return F.cross_entropy(logits.float().reshape(-1, logits.shape[-1]), labels.reshape(-1))


    @torch.no_grad()
    def sample(self, prompt, seq_len, temperature=1., filter_thres=0.9, use_cache_kv=False, use_graph=False):
        """Extend `prompt` to seq_len tokens and return the new ones (transformer.py:213-252).
        temperature <= 0 is greedy; otherwise gumbel sampling over the top (1 - filter_thres)
        share of the vocabulary.  With use_cache_kv every step after the first is a decode step;
        use_graph (with use_cache_kv, bf16 models) replays those steps from a captured HIP graph
        (decode_session.TransformerDecodeSession) instead of launching them one by one."""
        out, cache, session = prompt.clone(), None, None
        for _ in range(max(0, seq_len - prompt.shape[-1])):
            if session is not None:
                logits = session.step(out[:, -1:])
            else:
                logits, next_cache = self.forward(out, cache=cache, return_cache=True)
                if use_cache_kv:
                    cache = next_cache
                    if use_graph:
                        from .decode_session import TransformerDecodeSession
                        session = TransformerDecodeSession(self, cache, max_len=seq_len)
            logits = logits[:, -1].float()
            if temperature <= 0.:
                tok = logits.argmax(dim=-1, keepdim=True)
            else:
                kk = math.ceil((1 - filter_thres) * logits.shape[-1])
                val, ind = logits.topk(kk, dim=-1)
                logits = torch.full_like(logits, float('-inf')).scatter_(-1, ind, val)
                noise = -torch.log(-torch.log(torch.rand_like(logits).clamp_min(1e-20)).clamp_min(1e-20))
                tok = (logits / max(temperature, 1e-10) + noise).argmax(dim=-1, keepdim=True)
            out = torch.cat((out, tok), dim=-1)
        return out[..., prompt.shape[-1]:]
