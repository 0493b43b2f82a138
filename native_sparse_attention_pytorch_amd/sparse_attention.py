"""`SparseAttention` with the reference's constructor, parameter names and forward signature
(native_sparse_attention_pytorch/native_sparse_attention.py:188-336, 549-557), whose
training / prefill forward runs the four NSA subsystems as gfx950 HIP kernels:

  compressed attention + block-importance logits   ops.compress_attend     (NSA.py:621-691)
  importance softmax + top-k + slot mask            ops.importance_topk     (NSA.py:693-721)
  block-selection attention                         ops.native_sparse_attend(NSA.py:717-819)
  sliding-window attention                          ops.sliding_attend      (NSA.py:841-850)
  sigmoid strategy gate + head merge                ops.gate_combine        (NSA.py:854-860)

The dense projections (qkv, compression MLP, gate logits, output) stay `nn.Linear` GEMMs.  There
is no non-HIP path: CPU tensors, a missing library or an unsupported shape raise.

Single-token decoding over the caches (NSA.py:338-547) runs the same branches through
ops.decode_range_attend / ops.decode_select_attend.  The key / value and compressed caches the
module hands back are prefixes of buffers with spare capacity: the next step writes its row in
place instead of re-concatenating the whole cache (amortised O(1) per token rather than O(n)).
"""
from __future__ import annotations

from copy import deepcopy

import torch
import torch.nn.functional as F
from torch import nn

from . import ops


class RotaryEmbedding(nn.Module):
    """Rotary position embedding with the defaults of the package the reference imports
    (NSA.py:14, 238): theta 10000, feature pairs (2k, 2k+1), angles in fp32."""

    def __init__(self, dim: int, theta: float = 10000.0):
        super().__init__()
        self.freqs = nn.Parameter(1.0 / (theta ** (torch.arange(0, dim, 2).float() / dim)), requires_grad=False)

    def rotate(self, t: torch.Tensor, offset: int = 0) -> torch.Tensor:
        n = t.shape[-2]
        pos = torch.arange(offset, offset + n, device=t.device, dtype=torch.float32)
        ang = torch.outer(pos, self.freqs.float())
        cos, sin = ang.cos().repeat_interleave(2, dim=-1), ang.sin().repeat_interleave(2, dim=-1)
        tf = t.float()
        rot = torch.stack((-tf[..., 1::2], tf[..., 0::2]), dim=-1).flatten(-2)
        return (tf * cos + rot * sin).to(t.dtype)

    def rotate_queries_with_cached_keys(self, q, k):
        return self.rotate(q, offset=k.shape[-2] - q.shape[-2]), self.rotate(k)


def _append_rows(t: torch.Tensor, extra: int = 1, dtype=torch.bfloat16, min_capacity: int = 128, feat: int | None = None):
    """Grow the 'b h n d' cache `t` by `extra` rows.  Returns (view of n+extra rows, view of the
    new rows).  When `t` is the filled prefix of a buffer made here, the rows are taken from the
    buffer's spare capacity; otherwise (a cache from the parallel forward, a branch point that
    re-uses an older cache, no capacity left) the contents move to a new bf16 buffer of twice
    the size first, so a caller that keeps an old cache tuple never sees it change."""
    b, h, n, d = t.shape
    feat = d if feat is None else feat                # buffers may be wider than the rows handed in (zero-padded features)
    base = t._base
    ok = (base is not None and getattr(base, "_nsa_filled", -1) == n and base.dtype == dtype and d == feat
          and base.dim() == 4 and base.shape[2] >= n + extra and base.shape[:2] == t.shape[:2] and base.shape[3] == d
          and t.data_ptr() == base.data_ptr() and t.stride() == base.stride())
    if not ok:
        make = torch.empty if d == feat else torch.zeros
        base = make((b, h, max(2 * (n + extra), min_capacity), feat), dtype=dtype, device=t.device)
        base[:, :, :n, :d].copy_(t)
    base._nsa_filled = n + extra
    return base[:, :, :n + extra], base[:, :, n:n + extra]


class _FlattenWindow(nn.Module):
    def forward(self, x):                                   # 'b h w n d -> b h w (n d)'
        return x.flatten(-2)


class _GateLayout(nn.Module):
    def __init__(self, heads):
        super().__init__()
        self.heads = heads

    def forward(self, x):                                   # 'b n (h s) -> b h n s'
        b, n, _ = x.shape
        return x.reshape(b, n, self.heads, 3).permute(0, 2, 1, 3)


class SparseAttention(nn.Module):
    def __init__(
        self,
        dim,
        dim_head,
        heads,
        sliding_window_size,
        compress_block_size,
        compress_block_sliding_stride,
        selection_block_size,
        num_selected_blocks,
        kv_heads=None,
        num_compressed_mem_kv=1,
        causal=False,
        norm=True,
        use_diff_topk=False,
        use_triton_kernel=False,
        query_heads_share_selected_kv=True,
        compress_mlp: nn.Module | None = None,
        compress_mlp_expand_factor=1.0,
        strategy_combine_mlp: nn.Module | None = None,
    ):
        super().__init__()
        kv_heads = heads if kv_heads is None else kv_heads
        assert kv_heads <= heads and heads % kv_heads == 0
        self.heads, self.dim_head, self.kv_heads = heads, dim_head, kv_heads
        self.num_grouped_queries = heads // kv_heads
        self.scale = dim_head ** -0.5
        dim_inner, dim_kv_inner = dim_head * heads, dim_head * kv_heads
        self.norm = nn.RMSNorm(dim) if norm else nn.Identity()
        self.causal = causal
        self.rotary_emb = RotaryEmbedding(dim_head)
        self.qkv_split = (dim_inner, dim_kv_inner, dim_kv_inner)
        self.to_qkv = nn.Linear(dim, sum(self.qkv_split), bias=False)
        self.sliding_window_size = sliding_window_size

        self.compress_block_size = compress_block_size
        self.compress_block_sliding_stride = compress_block_sliding_stride
        assert compress_block_size >= compress_block_sliding_stride, 'compress_block_size must be >= compress_block_sliding_stride'
        assert compress_block_sliding_stride > 0, 'compress_block_sliding_stride must be greater than 0'
        assert selection_block_size % compress_block_sliding_stride == 0, \
            f'selection_block_size {selection_block_size} must be divisible by compress_block_sliding_stride {compress_block_sliding_stride}'

        assert num_compressed_mem_kv > 0
        self.num_mem_compress_kv = num_compressed_mem_kv
        self.compress_mem_kv = nn.Parameter(torch.zeros(2, kv_heads, num_compressed_mem_kv, dim_head))
        self.k_intrablock_positions = nn.Parameter(torch.zeros(kv_heads, compress_block_size, dim_head))
        self.v_intrablock_positions = nn.Parameter(torch.zeros(kv_heads, compress_block_size, dim_head))

        if compress_mlp is None:
            compress_dim = compress_block_size * dim_head
            hidden = int(compress_mlp_expand_factor * compress_dim)
            compress_mlp = nn.Sequential(_FlattenWindow(), nn.Linear(compress_dim, hidden), nn.ReLU(), nn.Linear(hidden, dim_head))
        self.k_compress = deepcopy(compress_mlp)
        self.v_compress = deepcopy(compress_mlp)

        self.use_diff_topk = use_diff_topk
        self.query_heads_share_selected_kv = query_heads_share_selected_kv
        self.selection_block_size = selection_block_size
        assert num_selected_blocks >= 0
        if num_selected_blocks == 0:
            print('`num_selected_blocks` should be set greater than 0, unless if you are ablating it for experimental purposes')
        self.num_selected_blocks = num_selected_blocks
        self.use_triton_kernel = use_triton_kernel      # kept for call-site compatibility; the HIP kernels always run
        # an fp32 module takes the fp32 forward kernels (agreement with the reference's fp32 path to 1e-5), in the parallel
        # forward - with or without gradients, whose values then come from the bf16 kernels - and in the decode step; with
        # this switched off its attention runs in bf16 like any other module's
        self.fp32_kernels = True

        if strategy_combine_mlp is None:
            strategy_combine_mlp = nn.Linear(dim, 3 * heads)
            nn.init.zeros_(strategy_combine_mlp.weight)
            strategy_combine_mlp.bias.data.copy_(torch.tensor([-2., -2., 2.] * heads))
        self.to_strategy_combine = nn.Sequential(strategy_combine_mlp, nn.Sigmoid(), _GateLayout(heads))
        self.combine_heads = nn.Linear(dim_inner, dim, bias=False)

    # the switch's earlier name
    fp32_inference_kernels = property(lambda self: self.fp32_kernels, lambda self, on: setattr(self, "fp32_kernels", bool(on)))

    # ------------------------------------------------------------------------------ pieces

    @classmethod
    def _linear(cls, layer, x):
        # a plain nn.Linear without hooks goes through ops.linear (its weight gradient fills the chip); anything else is called
        return ops.linear(x, layer.weight, layer.bias) if cls._plain(layer, nn.Linear) else layer(x)

    @staticmethod
    def _plain(layer, kind):
        """A library layer of exactly this kind on which nothing is hooked, neither on the instance nor globally: only then may
        its weights be used directly (any hook is skipped when the layer's own `__call__` is)."""
        from torch.nn.modules import module as M
        own = (layer._forward_hooks, layer._forward_pre_hooks, layer._backward_hooks, layer._backward_pre_hooks)
        glob = tuple(getattr(M, name, None) for name in ("_global_forward_hooks", "_global_forward_pre_hooks", "_global_backward_hooks",
                                                         "_global_backward_pre_hooks", "_global_forward_hooks_always_called"))
        return type(layer) is kind and not any(own) and not any(glob)

    def _front_is_one_node(self, inp):
        """Norm, qkv projection and gate logits as ops.normed_projections: a bf16 module with its default layers, under autograd."""
        norm, qkv, gate = self.norm, self.to_qkv, self.to_strategy_combine[0]
        if not (torch.is_grad_enabled() and inp.is_cuda and inp.dtype == torch.bfloat16 and not torch.compiler.is_compiling()):
            return False
        if not (self._plain(norm, nn.RMSNorm) and self._plain(qkv, nn.Linear) and self._plain(gate, nn.Linear)):
            return False
        if qkv.bias is not None or any(t is not None and t.dtype != torch.bfloat16 for t in (norm.weight, qkv.weight, gate.weight, gate.bias)):
            return False
        if tuple(norm.normalized_shape) != tuple(inp.shape[-1:]) or torch.is_autocast_enabled():
            return False
        return ops.rms_norm_supported(inp, norm.weight) and (inp.requires_grad or any(p.requires_grad for p in self.parameters()))

    def _normed(self, x):
        norm = self.norm
        if self._plain(norm, nn.RMSNorm) and tuple(norm.normalized_shape) == tuple(x.shape[-1:]) and ops.rms_norm_supported(x, norm.weight):
            return ops.rms_norm(x, norm.weight, norm.eps)
        return norm(x)

    @classmethod
    def _compress(cls, mlp, windows):
        # the default network (flatten, linear, relu, linear) layer by layer, so that its projections go through ops.linear
        if not cls._plain(mlp, nn.Sequential):
            return mlp(windows)
        for layer in mlp:
            windows = cls._linear(layer, windows)
        return windows

    def _split_heads(self, t):
        b, n, hd = t.shape
        return t.view(b, n, hd // self.dim_head, self.dim_head).permute(0, 2, 1, 3)

    @torch.no_grad()
    def forward_inference(self, inp, cache, return_cache=True):
        """One decode step (NSA.py:338-547): `inp` 'b 1 dim' is the token at position t = cached
        length; returns the output and the advanced caches."""
        assert self.causal, 'inference only relevant for autoregressive'
        if not inp.is_cuda:
            raise RuntimeError("SparseAttention runs on the GPU only (HIP kernels, no CPU fallback)")
        (cache_k, cache_v), ((cache_ck, cache_cv), (run_k, run_v)) = cache
        b, t = inp.shape[0], cache_k.shape[-2]
        st, cbs, B = self.compress_block_sliding_stride, self.compress_block_size, self.selection_block_size
        G, bf16 = self.num_grouped_queries, torch.bfloat16
        freqs = self.rotary_emb.freqs

        x = self.norm(inp)
        q, k, v = self.to_qkv(x).split(self.qkv_split, dim=-1)
        q, k, v = self._split_heads(q), self._split_heads(k), self._split_heads(v)
        if (self.fp32_kernels and q.dtype == torch.float32 and self.dim_head <= 128 and self.dim_head % 4 == 0
                and all(t.dtype == torch.float32 for t in (cache_k, cache_v, cache_ck, cache_cv, run_k, run_v))):
            return self._forward_inference_fp32(x, q, k, v, cache, return_cache)
        # head dimensions other than the kernels' 64 / 128 run zero-padded: caches and window rows are then kept D wide
        # (the padding features stay zero), the projections and the compression network see the first d features
        d, D = self.dim_head, ops._kernel_dim(self.dim_head)
        pad = (lambda u: u) if D == d else (lambda u: F.pad(u, (0, D - d)))
        q16, k16, v16 = pad(q.to(bf16)), pad(k.to(bf16)), pad(v.to(bf16))
        if D != d:
            freqs = F.pad(freqs.detach().float(), (0, (D - d) // 2))

        # raw tokens of the open compression window (not rotated, NSA.py:377-380) and the caches' new row
        run_k, rk_row = _append_rows(run_k, dtype=run_k.dtype, min_capacity=cbs, feat=D)
        run_v, rv_row = _append_rows(run_v, dtype=run_v.dtype, min_capacity=cbs, feat=D)
        fused_run = run_k.dtype == bf16 and run_v.dtype == bf16
        if not fused_run:
            rk_row[..., :d].copy_(k)
            rv_row[..., :d].copy_(v)
        keys, _ = _append_rows(cache_k, feat=D)
        vals, _ = _append_rows(cache_v, feat=D)

        # one library call for the attention part of the step: rotation of q / k and the new cache rows
        # (NSA.py:384-393), compressed branch over every cached compressed key (NSA.py:396-420), block
        # selection from its logits (NSA.py:448-476), selected blocks + own block (NSA.py:446-515), last
        # window + 1 keys (NSA.py:519-530), merge + sigmoid gate + head merge (NSA.py:534-545)
        nc = cache_ck.shape[-2]
        ck16 = cv16 = None
        if nc > 0:
            ck16 = pad(cache_ck if cache_ck.dtype == bf16 else cache_ck.to(bf16))
            cv16 = pad(cache_cv if cache_cv.dtype == bf16 else cache_cv.to(bf16))
        merged, _, _ = ops.decode_step(q16, k16, v16, freqs, t, keys, vals, ck16, cv16, pad(self.compress_mem_kv[0]), pad(self.compress_mem_kv[1]),
                                       rk_row if fused_run else None, rv_row if fused_run else None, self.to_strategy_combine[0](x),
                                       per_block=B // st, block=B, num_sel=self.num_selected_blocks,
                                       share=self.query_heads_share_selected_kv, window=self.sliding_window_size, scale=self.scale)

        # a compression window is complete: compress it, keep the overlap (NSA.py:422-441)
        ck, cv = cache_ck, cache_cv
        if run_k.shape[-2] % cbs == 0:
            next_ck = self.k_compress((run_k[..., :d] + self.k_intrablock_positions)[:, :, None])
            next_cv = self.v_compress((run_v[..., :d] + self.v_intrablock_positions)[:, :, None])
            run_k, run_v = run_k[..., st:, :], run_v[..., st:, :]
            ck, ck_row = _append_rows(cache_ck)
            cv, cv_row = _append_rows(cache_cv)
            ck_row.copy_(next_ck)
            cv_row.copy_(next_cv)

        if D != d:
            merged = merged.reshape(b, 1, self.heads, D)[..., :d].reshape(b, 1, self.heads * d)
        out = self.combine_heads(merged.to(x.dtype))
        if not return_cache:
            return out
        return out, ((keys, vals), ((ck, cv), (run_k, run_v)))

    def _forward_inference_fp32(self, x, q, k, v, cache, return_cache):
        """One decode step of an fp32 module over fp32 caches (as `_forward_fp32` hands them back), every attention branch
        through the fp32 kernels: the reference's own criterion - token-by-token decoding equals the parallel forward to 1e-5
        (tests/test_sparse_attn.py:50-91) - then holds for this module too.  Same steps as `forward_inference`."""
        (cache_k, cache_v), ((cache_ck, cache_cv), (run_k, run_v)) = cache
        b, t = x.shape[0], cache_k.shape[-2]
        st, cbs, B = self.compress_block_sliding_stride, self.compress_block_size, self.selection_block_size
        M, d, f32 = self.num_mem_compress_kv, self.dim_head, torch.float32
        rq, rk = self.rotary_emb.rotate(q, offset=t), self.rotary_emb.rotate(k, offset=t)
        run_k, rk_row = _append_rows(run_k, dtype=f32, min_capacity=cbs)
        run_v, rv_row = _append_rows(run_v, dtype=f32, min_capacity=cbs)
        rk_row.copy_(k)
        rv_row.copy_(v)
        keys, k_row = _append_rows(cache_k, dtype=f32)
        vals, v_row = _append_rows(cache_v, dtype=f32)
        k_row.copy_(rk)
        v_row.copy_(v)

        # compressed branch over every cached compressed key (NSA.py:396-420); none cached: the branch is zero
        nc = cache_ck.shape[-2]
        if nc > 0:
            ak = torch.cat((self.compress_mem_kv[0][None].expand(b, -1, -1, -1), cache_ck), dim=-2)
            av = torch.cat((self.compress_mem_kv[1][None].expand(b, -1, -1, -1), cache_cv), dim=-2)
            c_out, _ = ops.dense_attend_f32(q, ak, av, 1, False, 0, st, M)
        else:
            c_out = torch.zeros_like(q)

        # selected blocks + own block up to the token (NSA.py:446-515)
        imp = None
        if self.num_selected_blocks > 0 and nc > 0:
            imp = ops.importance_logits_f32(q, cache_ck, st, B, self.query_heads_share_selected_kv, False, mask_own=False)
        num_sel = min(self.num_selected_blocks, imp.shape[-1]) if imp is not None else 0
        if num_sel > 0:
            _, idx, fmask = ops.importance_topk(imp.contiguous(), num_sel)
        else:
            idx = torch.zeros((b, self.kv_heads, 1, 0), dtype=torch.int32, device=x.device)
            fmask = idx.bool()
        f_out = ops.native_sparse_attend_f32(rq, keys, vals, B, idx, fmask, include_block_causal=True, q_offset=t)
        # last window + 1 keys (NSA.py:519-530)
        s_out, _ = ops.dense_attend_f32(rq, keys, vals, 0, True, self.sliding_window_size, q_offset=t)

        # a compression window is complete: compress it, keep the overlap (NSA.py:422-441)
        ck, cv = cache_ck, cache_cv
        if run_k.shape[-2] % cbs == 0:
            next_ck = self.k_compress((run_k + self.k_intrablock_positions)[:, :, None])
            next_cv = self.v_compress((run_v + self.v_intrablock_positions)[:, :, None])
            run_k, run_v = run_k[..., st:, :], run_v[..., st:, :]
            ck, ck_row = _append_rows(cache_ck, dtype=f32)
            cv, cv_row = _append_rows(cache_cv, dtype=f32)
            ck_row.copy_(next_ck)
            cv_row.copy_(next_cv)

        gates = self.to_strategy_combine(x)                                   # 'b h 1 3' after the sigmoid
        merged = gates[..., 0:1] * c_out + gates[..., 1:2] * f_out + gates[..., 2:3] * s_out
        out = self.combine_heads(merged.permute(0, 2, 1, 3).reshape(b, 1, self.heads * d))
        if not return_cache:
            return out
        return out, ((keys, vals), ((ck, cv), (run_k, run_v)))

    def _forward_fp32(self, x, qkv, return_cache):
        """The parallel forward of an fp32 module: every attention branch through the fp32 kernels (ops.*_f32), the gate and
        the merge in fp32 torch - the same steps as `forward` (NSA.py:579-862).  Under autograd the values are still those of
        the fp32 kernels and each branch's gradient comes from the bf16 kernels (ops.fp32_value_bf16_grad); rotation and
        window split are then plain differentiable torch."""
        b, n, _ = x.shape
        st, cbs, B = self.compress_block_sliding_stride, self.compress_block_size, self.selection_block_size
        M, d = self.num_mem_compress_kv, self.dim_head
        causal, win, share = self.causal, self.sliding_window_size, self.query_heads_share_selected_kv
        q, k, v = qkv.split(self.qkv_split, dim=-1)
        q, k, v = self._split_heads(q), self._split_heads(k), self._split_heads(v)
        L = (n // st) * st
        recording = torch.is_grad_enabled() and (qkv.requires_grad or any(p.requires_grad for p in self.parameters()))
        if d in (64, 128) and not recording:
            _, rq, rk, _, kw, vw = ops.qkv_prep_f32(qkv, self.rotary_emb.freqs, self.k_intrablock_positions, self.v_intrablock_positions,
                                                    self.heads, self.kv_heads, d, cbs, st)
        else:
            rq, rk = self.rotary_emb.rotate(q), self.rotary_emb.rotate(k)
            def win_of(t, pos):
                if L == 0:                                                    # fewer tokens than one stride: no window yet
                    return t.new_zeros((b, t.shape[1], 0, cbs, d)) + pos[None, :, None]
                return F.pad(t[..., :L, :], (0, 0, cbs - st, 0)).unfold(2, cbs, st).permute(0, 1, 2, 4, 3) + pos[None, :, None]
            kw, vw = win_of(k, self.k_intrablock_positions), win_of(v, self.v_intrablock_positions)
        ck0, cv0 = self.k_compress(kw), self.v_compress(vw)
        ck = torch.cat((self.compress_mem_kv[0][None].expand(b, -1, -1, -1), ck0), dim=-2)
        cv = torch.cat((self.compress_mem_kv[1][None].expand(b, -1, -1, -1), cv0), dim=-2)
        nc = ck0.shape[-2]
        c_out = ops.fp32_value_bf16_grad(lambda q_, k_, v_: ops.dense_attend_f32(q_, k_, v_, 1, causal, 0, st, M)[0],
                                         lambda q_, k_, v_: ops.compress_attend(q_, k_, v_, M, st, causal)[0], q, ck, cv)
        imp = None
        if self.num_selected_blocks > 0 and nc > 0:
            imp = ops.importance_logits_f32(q, ck0, st, B, share, causal)
            if imp is not None and not self.use_diff_topk:
                imp = imp.detach()
        num_sel = min(self.num_selected_blocks, imp.shape[-1]) if imp is not None else 0
        gates = None
        if num_sel > 0:
            vals, idx, fmask = ops.importance_topk(imp.contiguous(), num_sel)
            if self.use_diff_topk:
                gates = vals + (1. - vals).detach()                              # straight-through gates (NSA.py:715)
            block_causal = causal
        elif causal:
            idx = torch.zeros((b, self.kv_heads, n, 0), dtype=torch.int32, device=x.device)
            fmask, block_causal = idx.bool(), True
        else:
            idx = (torch.arange(n, device=x.device, dtype=torch.int32) // B)[None, None, :, None].expand(b, self.kv_heads, n, 1).contiguous()
            fmask, block_causal = torch.ones_like(idx, dtype=torch.bool), False
        sel32 = lambda q_, k_, v_, *g_: ops.native_sparse_attend_f32(q_, k_, v_, B, idx, fmask, include_block_causal=block_causal)
        sel16 = lambda q_, k_, v_, *g_: ops.native_sparse_attend(q_, k_, v_, B, idx, fmask, sel_scale=g_[0] if g_ else None,
                                                                 include_block_causal=block_causal)
        f_out = ops.fp32_value_bf16_grad(sel32, sel16, rq, rk, v, *(() if gates is None else (gates,)))
        s_out = ops.fp32_value_bf16_grad(lambda q_, k_, v_: ops.dense_attend_f32(q_, k_, v_, 0, causal, win)[0],
                                         lambda q_, k_, v_: ops.sliding_attend(q_, k_, v_, win, causal=causal), rq, rk, v)
        gates3 = self.to_strategy_combine(x)                                  # 'b h n 3' after the sigmoid
        merged = gates3[..., 0:1] * c_out + gates3[..., 1:2] * f_out + gates3[..., 2:3] * s_out
        out = self.combine_heads(merged.permute(0, 2, 1, 3).reshape(b, n, self.heads * d))
        if not return_cache:
            return out
        co = cbs - st
        run_k, run_v = k, v
        if co > 0:
            run_k, run_v = F.pad(run_k, (0, 0, co, 0)), F.pad(run_v, (0, 0, co, 0))
        return out, ((rk, v), ((ck0, cv0), (run_k[..., L:, :], run_v[..., L:, :])))

    def forward(self, inp, cache=None, disable_triton_kernel=False, sliding_window_flex_mask=None,
                fine_selection_flex_mask=None, return_cache=False):
        if cache is not None:
            assert inp.shape[1] == 1, 'input must be single tokens if inferencing with cache key values'
            return self.forward_inference(inp, cache, return_cache=return_cache)
        assert not (not self.causal and return_cache)
        # sliding_window_flex_mask / fine_selection_flex_mask are the reference's precomputed flex-attention forms of the masks
        # this module's configuration already determines (NSA.py:40-109, 739, 839); the HIP kernels build those masks by index
        # arithmetic, so the arguments are accepted and not read
        if not inp.is_cuda:
            raise RuntimeError("SparseAttention runs on the GPU only (HIP kernels, no CPU fallback)")

        b, n, _ = inp.shape
        st, cbs, B = self.compress_block_sliding_stride, self.compress_block_size, self.selection_block_size
        M, G = self.num_mem_compress_kv, self.num_grouped_queries
        bf16 = torch.bfloat16

        logits = None
        if self._front_is_one_node(inp):
            x = None
            qkv, logits = ops.normed_projections(inp, self.norm.weight, self.norm.eps, self.to_qkv.weight,
                                                 self.to_strategy_combine[0].weight, self.to_strategy_combine[0].bias)
        else:
            x = self._normed(inp)
            qkv = self._linear(self.to_qkv, x)
        if (x is not None and self.fp32_kernels and qkv.dtype == torch.float32
                and self.dim_head <= 128 and self.dim_head % 4 == 0 and not torch.compiler.is_compiling()):
            return self._forward_fp32(x, qkv, return_cache)
        q, k, v = qkv.split(self.qkv_split, dim=-1)
        q, k, v = self._split_heads(q), self._split_heads(k), self._split_heads(v)      # views; read below only by the unfused path and the caches

        # compressed keys / values from the un-rotated k, v
        L = (n // st) * st
        fused = ops.qkv_prep_supported(qkv, self.dim_head)
        if fused:
            # head split, rotation of q / k (NSA.py:643), window gather + intra-window positions (NSA.py:589-603) and the
            # bf16 casts as one pass over the projection's output; its backward writes the projection's gradient directly
            q16, rq16, rk16, v16, kw, vw = ops.qkv_prep(qkv, self.rotary_emb.freqs, self.k_intrablock_positions, self.v_intrablock_positions,
                                                        self.heads, self.kv_heads, self.dim_head, cbs, st)
        else:
            # window gather + intra-window positions in one HIP kernel per tensor (NSA.py:589-603)
            kw, vw = ops.compress_windows_pair(k.to(bf16), v.to(bf16), self.k_intrablock_positions, self.v_intrablock_positions, cbs, st)
            kw, vw = kw.to(k.dtype), vw.to(v.dtype)
        ck0, cv0 = self._compress(self.k_compress, kw), self._compress(self.v_compress, vw)
        mem_k, mem_v = self.compress_mem_kv.to(ck0.dtype).unbind(0)       # unbind: its backward is one stack, not two zero-filled slices
        ck = torch.cat((mem_k[None].expand(b, -1, -1, -1), ck0), dim=-2)
        cv = torch.cat((mem_v[None].expand(b, -1, -1, -1), cv0), dim=-2)
        nc = ck0.shape[-2]

        want_sel = self.num_selected_blocks > 0 and nc > 0
        share = self.query_heads_share_selected_kv
        qc = q16 if fused else q.to(bf16)
        ck16, cv16 = ck.to(bf16), cv.to(bf16)
        npf = B // st
        num_sel = min(self.num_selected_blocks, nc // npf) if want_sel else 0
        vals = idx = fmask = None
        if num_sel > 0 and not self.use_diff_topk and ops.compress_topk_supported(qc, ck16, M, st, B, num_sel, share):
            # without differentiable top-k nothing but the selection reads the importance scores: the compressed forward makes
            # the selection itself and the scores never reach memory
            c_out, idx, fmask = ops.compress_attend_topk(qc, ck16, cv16, M, st, self.causal, B, num_sel)
        elif num_sel > 0:
            # the logits are written out (under a causal mask, without differentiable top-k, only the part of every row a
            # query can select from: logits and `prefix` stay together between these two calls)
            if self.use_diff_topk:
                c_out, imp = ops.compress_attend(qc, ck16, cv16, M, st, self.causal, sel_block=B, share=share)
                prefix = None
            else:
                c_out, imp, prefix = ops.compress_attend(qc, ck16, cv16, M, st, self.causal, sel_block=B, share=share, prefix_only=True)
            vals, idx, fmask = ops.importance_topk(imp, num_sel, prefix=prefix)
        else:
            c_out, _ = ops.compress_attend(qc, ck16, cv16, M, st, self.causal)

        if not fused:
            # rotary positions for the selection and sliding branches (NSA.py:643), one HIP kernel each
            rq16, rk16 = ops.rotary_pair(q.to(bf16), k.to(bf16), self.rotary_emb.freqs)
            v16 = v.to(bf16)

        if num_sel > 0:
            # straight-through gates (NSA.py:715): value 1, gradient flows into the importance scores
            gates = (vals + (1. - vals).detach()) if self.use_diff_topk else None
            f_out = ops.native_sparse_attend(rq16, rk16, v16, B, idx, fmask, sel_scale=gates, include_block_causal=self.causal)
        elif self.causal:
            # nothing selectable: block-diagonal causal attention (NSA.py:821-837)
            idx = torch.zeros((b, self.kv_heads, n, 0), dtype=torch.int32, device=inp.device)
            f_out = ops.native_sparse_attend(rq16, rk16, v16, B, idx, idx.bool(), include_block_causal=True)
        else:
            # non-causal: every query attends its whole own block
            own = (torch.arange(n, device=inp.device, dtype=torch.int32) // B)[None, None, :, None].expand(b, self.kv_heads, n, 1)
            f_out = ops.native_sparse_attend(rq16, rk16, v16, B, own.contiguous(), torch.ones_like(own, dtype=torch.bool),
                                             include_block_causal=False)

        s_out = ops.sliding_attend(rq16, rk16, v16, self.sliding_window_size, causal=self.causal)

        if logits is None:
            logits = self._linear(self.to_strategy_combine[0], x)
        merged = ops.gate_combine(logits, c_out, f_out, s_out)
        out = self._linear(self.combine_heads, merged.to(qkv.dtype))

        if not return_cache:
            return out
        co = cbs - st
        run_k, run_v = k, v
        if co > 0:
            run_k, run_v = F.pad(run_k, (0, 0, co, 0)), F.pad(run_v, (0, 0, co, 0))
        return out, ((rk16.to(k.dtype), v), ((ck0, cv0), (run_k[..., L:, :], run_v[..., L:, :])))
