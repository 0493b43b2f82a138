"""CPU oracle for the Native Sparse Attention hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package imports this file; it is
called from tests/, from __graft_entry__.smoke() and from the cpu_baseline leg of
bench.py, always as the checker and never as the thing being measured as product.

It restates, in plain PyTorch (CPU, any float dtype), the arithmetic of the
reference's pure-torch path (`use_triton_kernel=False`):

  native_sparse_attention_pytorch/native_sparse_attention.py
      :153-184  attend()                       -> attend
      :270-275  split_compress_window          -> compress_windows
      :549-867  SparseAttention.forward        -> SparseAttentionOracle.forward
      :338-547  forward_inference              -> SparseAttentionOracle.forward_inference
  native_sparse_attention_pytorch/transformer.py
      :254-330  Transformer.forward (+ caches) -> TransformerOracle.forward
      :213-252  Transformer.sample             -> TransformerOracle.sample
      :46-109   mask closed forms              -> sliding_mask / compress_mask / fine_mask
  test_triton_nsa.py:32-133 regular_attend     -> select_attend (functional contract of
                                                  native_sparse_attend, TRI.py:1938-1987)

What pins each function (see tests/test_oracle_*.py):
  attend / compressed branch  : F.scaled_dot_product_attention with the explicit mask
  compress_windows            : brute-force python loop on tiny shapes
  importance + top-k          : brute-force python loop restating NSA.py:652-713 term by
                                term; invariants (distinct, strictly-earlier blocks)
  select_attend (gather form) : dense-mask SDPA under fine_mask (NSA.py:90-104);
                                S=0 -> block-diagonal; S>=W -> full causal attention
  sliding_attend              : SDPA with the band mask (NSA.py:48-56); win>=n -> causal
  gate combine                : closed form at init (sigmoid([-2,-2,2]))
  forward_inference, caches   : the reference's own criterion (tests/test_sparse_attn.py:50-118):
                                token-by-token decode == parallel forward to 1e-5; greedy
                                sampling with and without caches gives the same tokens
  SparseAttentionOracle.forward (the wiring of the pieces above: which branch sees rotated q / k,
                                the gate fed by the normed input, memory slots first) and
  TransformerOracle.forward   : tests/test_oracle_composition.py - the module output rebuilt from
                                library attention under the three dense masks of NSA.py:46-109 with a
                                complex-multiplication rotary and python loops, no function of this
                                file; the transformer from its closed forms (depth 0, silenced
                                sub-layers, one hand-rolled layer, hand-written shifted cross entropy)

Two modes.  Called with fp32 (or fp64) parameters and inputs this file is the "truth" the HIP path is
compared with.  Cast to another dtype (`oracle.to(torch.bfloat16)`, bf16 input) it is the
dtype-faithful mode: every fill value (-finfo.max // 10, -finfo.max), the -1e3 pad, the softmaxes
and the GEMMs are evaluated in that dtype exactly as the reference's torch path does when its
module is cast (NSA.py:131-132, 171, 693, 742); tests use it to tell the error of the HIP kernels
from the error any bf16 run of the reference has (tests/test_module_gpu.py).

PARITY UNPINNED (third-party packages absent from the reference tree and from this
image, so no fixture can be produced): the numeric convention of
`rotary_embedding_torch.RotaryEmbedding` (theta=10000, interleaved pairs, fp32 angles,
restated in `rotary`) and the rounding order inside `local_attention.LocalAttention`
(q scaled before the dot; restated as a dense band mask in `sliding_attend`).  The
reference's own test (tests/test_sparse_attn.py:50-86) only fixes them up to
self-consistency.  torch.topk's tie order is likewise unpinned: this file resolves ties
towards the lower block index (stable sort), and slots whose value is not above the
1e-10 threshold are don't-care.
"""
from __future__ import annotations

import math
from copy import deepcopy

import torch
import torch.nn.functional as F
from torch import nn


# --------------------------------------------------------------------------- helpers

def _neg_max(t: torch.Tensor) -> float:
    return -torch.finfo(t.dtype).max


def split_heads(x: torch.Tensor, dim_head: int) -> torch.Tensor:
    b, n, hd = x.shape
    return x.reshape(b, n, hd // dim_head, dim_head).permute(0, 2, 1, 3)


def merge_heads(x: torch.Tensor) -> torch.Tensor:
    b, h, n, d = x.shape
    return x.permute(0, 2, 1, 3).reshape(b, n, h * d)


# ------------------------------------------------------------------- mask closed forms

def sliding_mask(n: int, window: int, causal: bool = True) -> torch.Tensor:
    """bool [n, n], True = attend.  NSA.py:48-56 (distance = i - j)."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    dist = i - j
    lo = 0 if causal else -window
    return (dist <= window) & (dist >= lo)


def compress_mask(n: int, num_compress: int, stride: int, num_mem: int = 1, causal: bool = True) -> torch.Tensor:
    """bool [n, num_mem + num_compress].  NSA.py:632-637 / :69-76: compressed key c is visible
    to query i iff its last covered token (c+1)*stride-1 < i; memory slots always."""
    if not causal:
        return torch.ones(n, num_mem + num_compress, dtype=torch.bool)
    last_tok = (torch.arange(num_compress) + 1) * stride - 1
    last_tok = torch.cat((torch.full((num_mem,), -1, dtype=last_tok.dtype), last_tok))
    return last_tok[None, :] < torch.arange(n)[:, None]


def fine_mask(idx: torch.Tensor, fmask: torch.Tensor, n: int, block: int, causal: bool = True) -> torch.Tensor:
    """Dense bool mask [b, h_sel, n, W*block] equivalent to the gather path.  NSA.py:90-104.
    idx / fmask: [b, h_sel, n, S]."""
    b, h, _, S = idx.shape
    W = math.ceil(n / block)
    onehot = torch.zeros(b, h, n, W, dtype=torch.bool)
    if S > 0:
        # a block is attended if any slot that names it has fmask True
        cnt = torch.zeros(b, h, n, W, dtype=torch.int32)
        cnt.scatter_add_(-1, idx.long(), fmask.to(torch.int32))
        onehot = cnt > 0
    sel = onehot.repeat_interleave(block, dim=-1)            # [b,h,n,W*block]
    if not causal:
        return sel
    i = torch.arange(n)[:, None]
    j = torch.arange(W * block)[None, :]
    return (i >= j) & ((i // block == j // block) | sel)


# ------------------------------------------------------------------------------ rotary

class RotaryEmbedding(nn.Module):
    """Restatement of rotary_embedding_torch.RotaryEmbedding(dim) defaults (PARITY UNPINNED,
    package absent): inv_freq_k = 10000^(-2k/dim); features (2k, 2k+1) form a pair; angles in
    fp32; result cast back to the input dtype.  Used at NSA.py:238, 643."""

    def __init__(self, dim: int, theta: float = 10000.0):
        super().__init__()
        freqs = 1.0 / (theta ** (torch.arange(0, dim, 2).float() / dim))
        self.freqs = nn.Parameter(freqs, requires_grad=False)

    def rotate(self, t: torch.Tensor, offset: int = 0) -> torch.Tensor:
        n = t.shape[-2]
        pos = torch.arange(n, device=t.device, dtype=torch.float32) + offset
        ang = pos[:, None] * self.freqs.float()[None, :]          # [n, d/2]
        ang = ang.repeat_interleave(2, dim=-1)                    # [n, d]
        tf = t.float()
        x1, x2 = tf[..., 0::2], tf[..., 1::2]
        rot = torch.stack((-x2, x1), dim=-1).flatten(-2)
        return (tf * ang.cos() + rot * ang.sin()).to(t.dtype)

    def rotate_queries_with_cached_keys(self, q, k):
        return self.rotate(q, offset=k.shape[-2] - q.shape[-2]), self.rotate(k)


# ------------------------------------------------------------------------------ attend

def attend(q, k, v, mask=None, return_sim=False, scale=None):
    """GQA softmax attention, NSA.py:153-184.  q [b,Hq,i,d], k/v [b,Hkv,j,d]; query head hq
    uses kv head hq // G.  Masked logits are filled with -finfo.max // 10 (NSA.py:171)."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    b, hq, i, d = q.shape
    hk = k.shape[1]
    g = hq // hk
    qg = q.reshape(b, hk, g, i, d)
    sim = torch.einsum('bhgid,bhjd->bhgij', qg, k) * scale
    if mask is not None:
        sim = sim.masked_fill(~mask, _neg_max(sim) // 10)
    attn = sim.softmax(dim=-1)
    out = torch.einsum('bhgij,bhjd->bhgid', attn, v).reshape(b, hq, i, v.shape[-1])
    if not return_sim:
        return out
    return out, sim.reshape(b, hq, i, -1)


# --------------------------------------------------------------------- compress windows

def compress_windows(t: torch.Tensor, block: int, stride: int) -> torch.Tensor:
    """[b,h,L,d] with L % stride == 0 -> [b,h,L/stride,block,d]; window w holds tokens
    [(w+1)*stride-block, (w+1)*stride), zeros left of token 0.  NSA.py:270-275."""
    b, h, L, d = t.shape
    if L == 0:
        return t.reshape(b, h, 0, block, d)
    padded = F.pad(t, (0, 0, block - stride, 0))
    return padded.unfold(2, block, stride).permute(0, 1, 2, 4, 3).contiguous()


class _FlattenWindow(nn.Module):
    def forward(self, x):                                        # [b,h,w,n,d] -> [b,h,w,n*d]
        return x.flatten(-2)


# ------------------------------------------------------------ importance scores + top-k

def importance_logits(csim, num_mem, g, share, stride, block):
    """NSA.py:652-691: block-importance logits before the padded softmax.  csim [b,Hq,n,num_mem+Nc]
    = scaled, masked compressed logits.  Returns [b,H_sel,n,nb] (nb may be 0); invisible keys carry
    the reference's fill (-finfo.max/10, averaged), the query's own block -finfo.max."""
    imp = csim[..., num_mem:]
    b, hq, n, nc = imp.shape
    if share:
        imp = imp.reshape(b, hq // g, g, n, nc).mean(dim=2)
    if stride != block:
        npf = block // stride
        keep = (nc // npf) * npf
        imp = imp[..., :keep]
        if imp.numel() > 0:
            imp = imp.reshape(*imp.shape[:-1], keep // npf, npf).mean(dim=-1)
            nb = imp.shape[-1]
            own = (torch.arange(n)[:, None] // block) == torch.arange(nb)[None, :]
            imp = imp.masked_fill(own, _neg_max(csim))
    return imp


def importance_softmax(logits):
    """NSA.py:693-695: left-pad one column of -1e3, softmax, drop the column."""
    imp = F.pad(logits, (1, 0), value=-1e3)
    return imp.softmax(dim=-1)[..., 1:]


def importance_from_csim(csim, num_mem, g, share, stride, block):
    return importance_softmax(importance_logits(csim, num_mem, g, share, stride, block))


def topk_lower_index_first(scores: torch.Tensor, k: int):
    """torch.topk semantics (values descending) with ties resolved towards the lower index.
    NSA.py:713."""
    order = torch.sort(scores, dim=-1, descending=True, stable=True)
    return order.values[..., :k], order.indices[..., :k]


# --------------------------------------------------------- selection (fine) attention

def select_attend(q, k, v, idx, fmask, block, causal=True, gates=None, return_lse=False, chunk=256, q_offset=0):
    """Block-selection attention in gather form.  NSA.py:741-819, test_triton_nsa.py:32-133.

    q [b,Hq,n,d]; k,v [b,Hkv,n,d]; idx,fmask [b,Hsel,n,S] with Hsel in (Hkv, Hq).
    Each query attends (softmax over the concatenation) to the `block` keys of every
    selected block whose slot mask is True - with NO causal mask inside selected blocks and
    duplicates counted once per slot - plus, when `causal`, its own block under a
    lower-triangular mask.  `gates` [b,Hsel,n,S] multiplies the selected keys (NSA.py:793-797).
    Chunked over queries; mathematically identical to the reference's one-shot gather.
    `q_offset`: q/idx/fmask hold only the queries at positions q_offset .. q_offset+len-1 of
    the sequence k/v span (used to time or check a slice of a long sequence).
    """
    b, hq, nq, d = q.shape
    n = k.shape[2]
    hk = k.shape[1]
    hs = idx.shape[1]
    S = idx.shape[-1]
    if hs != hk:                                  # per-query-head selection: G becomes 1
        k = k.repeat_interleave(hq // hk, dim=1)
        v = v.repeat_interleave(hq // hk, dim=1)
        hk = hq
    g = hq // hk
    W = math.ceil(n / block)
    pad = W * block - n
    scale = d ** -0.5
    kp = F.pad(k, (0, 0, 0, pad)).reshape(b, hk, W, block, d)
    vp = F.pad(v, (0, 0, 0, pad)).reshape(b, hk, W, block, d)
    out = torch.empty_like(q)
    lse = torch.empty(b, hq, nq, dtype=torch.float32)
    tril = torch.ones(block, block, dtype=torch.bool).tril()
    bi = torch.arange(b)[:, None, None, None]
    hi = torch.arange(hk)[None, :, None, None]
    for s0 in range(0, nq, chunk):
        s1 = min(nq, s0 + chunk)
        c = s1 - s0
        pos = torch.arange(s0, s1) + q_offset
        ci = idx[:, :, s0:s1].long()                                    # [b,hk,c,S]
        cm = fmask[:, :, s0:s1]
        cg = gates[:, :, s0:s1] if gates is not None else None
        if causal:
            own = (pos // block)[None, None, :, None].expand(b, hk, c, 1)
            ci = torch.cat((ci, own), dim=-1)
            cm = cm[..., None].expand(b, hk, c, S, block)
            cm = torch.cat((cm, tril[pos % block][None, None, :, None, :].expand(b, hk, c, 1, block)), dim=-2)
            if cg is not None:
                cg = F.pad(cg, (0, 1), value=1.0)
        else:
            cm = cm[..., None].expand(b, hk, c, S, block)
        gk = kp[bi, hi, ci]                                              # [b,hk,c,S',block,d]
        gv = vp[bi, hi, ci]
        if cg is not None:
            gk = gk * cg[..., None, None]
        Sx = ci.shape[-1]
        gk = gk.reshape(b, hk, c, Sx * block, d)
        gv = gv.reshape(b, hk, c, Sx * block, d)
        cm = cm.reshape(b, hk, 1, c, Sx * block)
        qc = q[:, :, s0:s1].reshape(b, hk, g, c, d)
        sim = torch.einsum('bhgid,bhijd->bhgij', qc, gk) * scale
        sim = sim.masked_fill(~cm, _neg_max(sim))
        attn = sim.softmax(dim=-1)
        out[:, :, s0:s1] = torch.einsum('bhgij,bhijd->bhgid', attn, gv).reshape(b, hq, c, d)
        lse[:, :, s0:s1] = torch.logsumexp(sim.float(), dim=-1).reshape(b, hq, c)
    if return_lse:
        return out, lse
    return out


def block_local_attend(q, k, v, block, causal):
    """Fallback when nothing can be selected: attention inside each fine block only.
    NSA.py:821-837."""
    b, hq, n, d = q.shape
    W = math.ceil(n / block)
    pad = W * block - n
    def blk(t):
        h = t.shape[1]
        t = F.pad(t, (0, 0, 0, pad)).reshape(b, h, W, block, d)
        return t.permute(0, 2, 1, 3, 4).reshape(b * W, h, block, d)
    m = torch.ones(block, block, dtype=torch.bool).tril() if causal else None
    o = attend(blk(q), blk(k), blk(v), mask=m)
    o = o.reshape(b, W, hq, block, d).permute(0, 2, 1, 3, 4).reshape(b, hq, W * block, d)
    return o[..., :n, :]


# ------------------------------------------------------------------- sliding attention

def sliding_attend(q, k, v, window, causal=True, chunk=1024):
    """Dense-mask restatement of LocalAttention(window_size=window, causal, exact_windowsize,
    autopad) as called at NSA.py:250-257, 841-850 (PARITY UNPINNED for rounding order): query i
    attends keys with 0 <= i-j <= window (causal) or |i-j| <= window.  q [b,Hq,n,d], k/v
    [b,Hkv,n,d] (GQA by kv-head-major grouping, equal to the reference's repeat)."""
    b, hq, n, d = q.shape
    hk = k.shape[1]
    g = hq // hk
    scale = d ** -0.5
    out = torch.empty_like(q)
    for s0 in range(0, n, chunk):
        s1 = min(n, s0 + chunk)
        lo = max(0, s0 - window)
        hi = s1 if causal else min(n, s1 + window)
        i = torch.arange(s0, s1)[:, None]
        j = torch.arange(lo, hi)[None, :]
        dist = i - j
        m = (dist <= window) & (dist >= (0 if causal else -window))
        qc = (q[:, :, s0:s1] * scale).reshape(b, hk, g, s1 - s0, d)
        sim = torch.einsum('bhgid,bhjd->bhgij', qc, k[:, :, lo:hi])
        sim = sim.masked_fill(~m, _neg_max(sim))
        attn = sim.softmax(dim=-1)
        out[:, :, s0:s1] = torch.einsum('bhgij,bhjd->bhgid', attn, v[:, :, lo:hi]).reshape(b, hq, s1 - s0, d)
    return out


# --------------------------------------------------------------------------- the module

class SparseAttentionOracle(nn.Module):
    """Restatement of SparseAttention (NSA.py:188-336 construction, :549-867 forward) with
    identical constructor arguments, parameter names and creation order, plus the
    single-token decode step over the three caches (NSA.py:338-547).  The decode restatement
    is pinned by the reference's own criterion (tests/test_sparse_attn.py:50-86): token-by-
    token outputs equal the parallel forward to 1e-5 in fp32."""

    def __init__(self, dim, dim_head, heads, sliding_window_size, compress_block_size,
                 compress_block_sliding_stride, selection_block_size, num_selected_blocks,
                 kv_heads=None, num_compressed_mem_kv=1, causal=False, norm=True,
                 use_diff_topk=False, use_triton_kernel=False, query_heads_share_selected_kv=True,
                 compress_mlp=None, compress_mlp_expand_factor=1.0, strategy_combine_mlp=None):
        super().__init__()
        kv_heads = heads if kv_heads is None else kv_heads
        assert kv_heads <= heads and heads % kv_heads == 0
        self.heads, self.kv_heads, self.dim_head = heads, kv_heads, dim_head
        self.num_grouped_queries = heads // kv_heads
        self.scale = dim_head ** -0.5
        self.causal = causal
        self.norm = nn.RMSNorm(dim) if norm else nn.Identity()
        self.rotary_emb = RotaryEmbedding(dim_head)
        self.qkv_split = (dim_head * heads, dim_head * kv_heads, dim_head * kv_heads)
        self.to_qkv = nn.Linear(dim, sum(self.qkv_split), bias=False)
        self.sliding_window_size = sliding_window_size
        assert compress_block_size >= compress_block_sliding_stride > 0
        assert selection_block_size % compress_block_sliding_stride == 0
        self.compress_block_size = compress_block_size
        self.compress_block_sliding_stride = compress_block_sliding_stride
        assert num_compressed_mem_kv > 0
        self.num_mem_compress_kv = num_compressed_mem_kv
        self.compress_mem_kv = nn.Parameter(torch.zeros(2, kv_heads, num_compressed_mem_kv, dim_head))
        self.k_intrablock_positions = nn.Parameter(torch.zeros(kv_heads, compress_block_size, dim_head))
        self.v_intrablock_positions = nn.Parameter(torch.zeros(kv_heads, compress_block_size, dim_head))
        if compress_mlp is None:
            cdim = compress_block_size * dim_head
            hidden = int(compress_mlp_expand_factor * cdim)
            compress_mlp = nn.Sequential(_FlattenWindow(), nn.Linear(cdim, hidden), nn.ReLU(), nn.Linear(hidden, dim_head))
        self.k_compress = deepcopy(compress_mlp)
        self.v_compress = deepcopy(compress_mlp)
        self.use_diff_topk = use_diff_topk
        self.query_heads_share_selected_kv = query_heads_share_selected_kv
        self.selection_block_size = selection_block_size
        assert num_selected_blocks >= 0
        self.num_selected_blocks = num_selected_blocks
        if strategy_combine_mlp is None:
            strategy_combine_mlp = nn.Linear(dim, 3 * heads)
            nn.init.zeros_(strategy_combine_mlp.weight)
            strategy_combine_mlp.bias.data.copy_(torch.tensor([-2.0, -2.0, 2.0] * heads))
        self.to_strategy_combine = nn.Sequential(strategy_combine_mlp, nn.Sigmoid())
        self.combine_heads = nn.Linear(dim_head * heads, dim, bias=False)

    # -- pieces, exposed so tests can compare intermediate tensors with the HIP path --

    def project(self, inp):
        x = self.norm(inp)
        q, k, v = self.to_qkv(x).split(self.qkv_split, dim=-1)
        return x, split_heads(q, self.dim_head), split_heads(k, self.dim_head), split_heads(v, self.dim_head)

    def compress(self, k, v):
        st, cbs = self.compress_block_sliding_stride, self.compress_block_size
        b, n = k.shape[0], k.shape[2]
        L = (n // st) * st
        kw = compress_windows(k[..., :L, :], cbs, st)
        vw = compress_windows(v[..., :L, :], cbs, st)
        if kw.numel() > 0:
            kw = kw + self.k_intrablock_positions[None, :, None]
            vw = vw + self.v_intrablock_positions[None, :, None]
        ck, cv = self.k_compress(kw), self.v_compress(vw)
        mem_k, mem_v = self.compress_mem_kv[0], self.compress_mem_kv[1]
        ck = torch.cat((mem_k[None].expand(b, -1, -1, -1), ck), dim=-2)
        cv = torch.cat((mem_v[None].expand(b, -1, -1, -1), cv), dim=-2)
        return ck, cv

    def select(self, csim):
        """importance -> (values, indices) or None when nothing can be selected."""
        nc = csim.shape[-1] - self.num_mem_compress_kv
        num_sel = min(self.num_selected_blocks, nc)
        if num_sel <= 0:
            return None
        imp = importance_from_csim(csim, self.num_mem_compress_kv, self.num_grouped_queries,
                                   self.query_heads_share_selected_kv,
                                   self.compress_block_sliding_stride, self.selection_block_size)
        num_sel = min(num_sel, imp.shape[-1])
        if num_sel <= 0:
            return None
        return topk_lower_index_first(imp, num_sel)

    def forward(self, inp, return_parts=False, selection_override=None, cache=None, return_cache=False):
        """selection_override = (idx, fmask) replaces the module's own top-k result (used to
        compare implementations under an identical discrete selection).  With `cache` the
        input is one token and the decode step runs (NSA.py:559-563)."""
        if cache is not None:
            assert inp.shape[1] == 1
            return self.forward_inference(inp, cache, return_cache=return_cache, selection_override=selection_override)
        assert self.causal or not return_cache
        b, n, _ = inp.shape
        st, B = self.compress_block_sliding_stride, self.selection_block_size
        x, q, k, v = self.project(inp)
        ck, cv = self.compress(k, v)
        nc = ck.shape[-2] - self.num_mem_compress_kv
        cmask = compress_mask(n, nc, st, self.num_mem_compress_kv, True) if self.causal else None
        c_out, csim = attend(q, ck, cv, mask=cmask, return_sim=True)
        rq, rk = self.rotary_emb.rotate_queries_with_cached_keys(q, k)
        sel = self.select(csim)
        if selection_override is not None:
            # the discrete choice comes from outside; values (for the gates) are re-read from this
            # module's own importance scores at the given indices
            idx, live = selection_override
            imp = importance_from_csim(csim, self.num_mem_compress_kv, self.num_grouped_queries,
                                       self.query_heads_share_selected_kv, st, B)
            vals = imp.gather(-1, idx.long())
            gates = (vals + (1.0 - vals).detach()) if self.use_diff_topk else None
            f_out = select_attend(rq, rk, v, idx, live, B, causal=self.causal, gates=gates)
        elif sel is not None:
            vals, idx = sel
            gates = (vals + (1.0 - vals).detach()) if self.use_diff_topk else None
            f_out = select_attend(rq, rk, v, idx, vals > 1e-10, B, causal=self.causal, gates=gates)
        else:
            vals = idx = None
            f_out = block_local_attend(rq, rk, v, B, self.causal)
        s_out = sliding_attend(rq, rk, v, self.sliding_window_size, causal=self.causal)
        gate = self.to_strategy_combine(x).reshape(b, n, self.heads, 3).permute(0, 2, 1, 3)
        out = gate[..., 0:1] * c_out + gate[..., 1:2] * f_out + gate[..., 2:3] * s_out
        y = self.combine_heads(merge_heads(out))
        if return_parts:
            return y, dict(q=q, k=k, v=v, rq=rq, rk=rk, ck=ck, cv=cv, csim=csim, c_out=c_out,
                           idx=idx, vals=vals, f_out=f_out, s_out=s_out, gate=gate)
        if return_cache:
            # NSA.py:605-619, 863-867: rotated keys and values; compressed keys without the
            # memory slots; the raw tokens after the last complete stride, preceded by the
            # window overlap (zeros left of token 0)
            M, cbs = self.num_mem_compress_kv, self.compress_block_size
            L = (n // st) * st
            run_k = F.pad(k, (0, 0, cbs - st, 0))[..., L:, :]
            run_v = F.pad(v, (0, 0, cbs - st, 0))[..., L:, :]
            return y, ((rk, v), ((ck[..., M:, :], cv[..., M:, :]), (run_k, run_v)))
        return y

    def forward_inference(self, inp, cache, return_cache=True, selection_override=None):
        """One decode step (NSA.py:338-547).  inp [b,1,dim]; cache as returned by `forward`.
        The token at position t = cached length attends to: every cached compressed key (plus the
        memory slots, unless there is none cached: then that branch is zero); the top blocks
        by importance plus the keys of its own block up to itself; its last window+1 keys."""
        assert self.causal
        (cache_k, cache_v), ((ck, cv), (run_k, run_v)) = cache
        b, t = inp.shape[0], cache_k.shape[-2]
        G, B, st, cbs, M = self.num_grouped_queries, self.selection_block_size, self.compress_block_sliding_stride, self.compress_block_size, self.num_mem_compress_kv
        x, q, k, v = self.project(inp)
        run_k, run_v = torch.cat((run_k, k), dim=-2), torch.cat((run_v, v), dim=-2)     # un-rotated (NSA.py:377-380)
        rq, rk = self.rotary_emb.rotate(q, offset=t), self.rotary_emb.rotate(k, offset=t)
        keys, vals_ = torch.cat((cache_k, rk), dim=-2), torch.cat((cache_v, v), dim=-2)

        # compressed branch (NSA.py:396-420): no mask, every cached block is complete
        nc = ck.shape[-2]
        if nc > 0:
            ak = torch.cat((self.compress_mem_kv[0][None].expand(b, -1, -1, -1), ck), dim=-2)
            av = torch.cat((self.compress_mem_kv[1][None].expand(b, -1, -1, -1), cv), dim=-2)
            csim = torch.einsum('bhgd,bhjd->bhgj', q.reshape(b, self.kv_heads, G, -1), ak) * self.scale
            c_out = torch.einsum('bhgj,bhjd->bhgd', csim.softmax(dim=-1), av).reshape(b, self.heads, 1, -1)
            imp = csim[..., M:]                                                        # [b, hk, G, nc]
        else:
            c_out = torch.zeros_like(q)
            imp = q.new_zeros(b, self.kv_heads, G, 0)

        # a window of cbs raw tokens is complete: compress it and keep the overlap (NSA.py:422-441)
        if run_k.shape[-2] % cbs == 0:
            nk = self.k_compress((run_k + self.k_intrablock_positions)[:, :, None])
            nv = self.v_compress((run_v + self.v_intrablock_positions)[:, :, None])
            keep = cbs - st
            run_k, run_v = run_k[..., cbs - keep:, :], run_v[..., cbs - keep:, :]
            ck, cv = torch.cat((ck, nk), dim=-2), torch.cat((cv, nv), dim=-2)

        # selection branch (NSA.py:446-515)
        npf = B // st
        nb = nc // npf if st != B else nc
        imp = imp[..., :nb * npf].reshape(b, self.kv_heads, G, nb, npf).mean(dim=-1) if st != B else imp
        num_sel = min(self.num_selected_blocks, nb)
        own = (t % B) + 1                                                              # keys of the own block, itself included
        seg_k, seg_v = [keys[..., -own:, :]], [vals_[..., -own:, :]]
        live = None
        qg = rq.reshape(b, self.kv_heads, G, -1)
        if num_sel > 0:
            if self.query_heads_share_selected_kv:
                imp = imp.mean(dim=2, keepdim=True)                                    # [b, hk, 1, nb]
            probs = F.pad(imp, (1, 0), value=-1e3).softmax(dim=-1)[..., 1:]
            if selection_override is not None:
                idx, lv = selection_override
                idx, lv = idx.reshape(probs.shape[:-1] + (-1,)).long(), lv.reshape(probs.shape[:-1] + (-1,))
            else:
                sv, idx = topk_lower_index_first(probs, num_sel)
                lv = sv > 1e-10
            W = -(-(t + 1) // B)
            kb = F.pad(keys, (0, 0, 0, W * B - (t + 1))).reshape(b, self.kv_heads, 1, W, B, -1)
            vb = F.pad(vals_, (0, 0, 0, W * B - (t + 1))).reshape(b, self.kv_heads, 1, W, B, -1)
            gi = idx[..., None, None].expand(-1, -1, -1, -1, B, kb.shape[-1])
            sk = kb.expand(-1, -1, idx.shape[2], -1, -1, -1).gather(3, gi).flatten(3, 4)   # [b, hk, 1|G, sel*B, d]
            sv_ = vb.expand(-1, -1, idx.shape[2], -1, -1, -1).gather(3, gi).flatten(3, 4)
            live = torch.cat((lv.repeat_interleave(B, dim=-1), lv.new_ones(lv.shape[:-1] + (own,))), dim=-1)
            fk = torch.cat((sk, seg_k[0][:, :, None].expand(-1, -1, sk.shape[2], -1, -1)), dim=-2)
            fv = torch.cat((sv_, seg_v[0][:, :, None].expand(-1, -1, sk.shape[2], -1, -1)), dim=-2)
            fsim = torch.einsum('bhgd,bhgjd->bhgj', qg, fk.expand(-1, -1, G, -1, -1)) * self.scale
            fsim = fsim.masked_fill(~live.expand_as(fsim), _neg_max(fsim))
            f_out = torch.einsum('bhgj,bhgjd->bhgd', fsim.softmax(dim=-1), fv.expand(-1, -1, G, -1, -1))
        else:
            fsim = torch.einsum('bhgd,bhjd->bhgj', qg, seg_k[0]) * self.scale
            f_out = torch.einsum('bhgj,bhjd->bhgd', fsim.softmax(dim=-1), seg_v[0])
        f_out = f_out.reshape(b, self.heads, 1, -1)

        # sliding branch (NSA.py:519-530): the last window+1 keys
        wk, wv = keys[..., -(self.sliding_window_size + 1):, :], vals_[..., -(self.sliding_window_size + 1):, :]
        ssim = torch.einsum('bhgd,bhjd->bhgj', qg, wk) * self.scale
        s_out = torch.einsum('bhgj,bhjd->bhgd', ssim.softmax(dim=-1), wv).reshape(b, self.heads, 1, -1)

        gate = self.to_strategy_combine(x).reshape(b, 1, self.heads, 3).permute(0, 2, 1, 3)
        out = gate[..., 0:1] * c_out + gate[..., 1:2] * f_out + gate[..., 2:3] * s_out
        y = self.combine_heads(merge_heads(out))
        if not return_cache:
            return y
        return y, ((keys, vals_), ((ck, cv), (run_k, run_v)))


def gate_combine(logits, c_out, f_out, s_out):
    """NSA.py:323-327, 854-856.  logits [b,n,3*Hq] (column h*3+s, s = compressed, selected,
    sliding); branches [b,Hq,n,d] -> [b,n,Hq*d]."""
    b, n, _ = logits.shape
    h = c_out.shape[1]
    g = torch.sigmoid(logits).reshape(b, n, h, 3).permute(0, 2, 1, 3)
    return merge_heads(g[..., 0:1] * c_out + g[..., 1:2] * f_out + g[..., 2:3] * s_out)


# --------------------------------------------------------------- training-step harness

def _feed_forward(dim, expansion_factor=4.0):
    hidden = int(dim * expansion_factor)
    return nn.Sequential(nn.RMSNorm(dim), nn.Linear(dim, hidden), nn.GELU(), nn.Linear(hidden, dim))


class TransformerOracle(nn.Module):
    """Restatement of the reference's training forward, transformer.py:142-211 (construction
    order: token_emb, per layer [attention, feed-forward], norm, to_logits) and :254-330
    (ids[:, :-1] -> logits, cross entropy against ids[:, 1:]; with a cache only the last token
    is embedded and every layer takes its decode step), and of greedy / temperature sampling
    with or without the caches (transformer.py:213-252)."""

    def __init__(self, num_tokens, dim, depth, dim_head=64, heads=8, kv_heads=None, ff_expansion_factor=4.0,
                 causal=True, sparse_attn_kwargs=None):
        super().__init__()
        self.token_emb = nn.Embedding(num_tokens, dim)
        layers = []
        for _ in range(depth):
            attn = SparseAttentionOracle(dim=dim, dim_head=dim_head, heads=heads, kv_heads=kv_heads, causal=causal, **sparse_attn_kwargs)
            layers.append(nn.ModuleList([attn, _feed_forward(dim, ff_expansion_factor)]))
        self.layers = nn.ModuleList(layers)
        self.norm = nn.RMSNorm(dim)
        self.to_logits = nn.Linear(dim, num_tokens, bias=False)

    def forward(self, ids, return_loss=False, cache=None, return_cache=False):
        if return_loss:
            ids, labels = ids[:, :-1], ids[:, 1:]
        tokens = self.token_emb(ids if cache is None else ids[:, -1:])
        layer_caches = iter(cache or [])
        next_cache = []
        for attn, ff in self.layers:
            if return_cache or cache is not None:
                attn_out, lc = attn(tokens, cache=next(layer_caches, None), return_cache=True)
                next_cache.append(lc)
            else:
                attn_out = attn(tokens)
            tokens = attn_out + tokens
            tokens = ff(tokens) + tokens
        logits = self.to_logits(self.norm(tokens))
        if not return_loss:
            return (logits, next_cache) if return_cache else logits
        return F.cross_entropy(logits.transpose(1, 2), labels)

    @torch.no_grad()
    def sample(self, prompt, seq_len, temperature=1.0, filter_thres=0.9, use_cache_kv=False):
        """transformer.py:213-252: extend `prompt` to seq_len tokens; temperature <= 0 is greedy,
        otherwise gumbel sampling over the top (1 - filter_thres) share of the vocabulary
        (transformer.py:45-62).  Returns only the new tokens."""
        out, cache = prompt.clone(), None
        for _ in range(max(0, seq_len - prompt.shape[-1])):
            logits, next_cache = self.forward(out, cache=cache, return_cache=True)
            if use_cache_kv:
                cache = next_cache
            logits = logits[:, -1]
            if temperature <= 0.0:
                tok = logits.argmax(dim=-1, keepdim=True)
            else:
                kk = math.ceil((1.0 - filter_thres) * logits.shape[-1])
                val, ind = logits.topk(kk, dim=-1)
                logits = torch.full_like(logits, float('-inf')).scatter(-1, ind, val)
                noise = -torch.log(-torch.log(torch.rand_like(logits).clamp_min(1e-20)).clamp_min(1e-20))
                tok = (logits / max(temperature, 1e-10) + noise).argmax(dim=-1, keepdim=True)
            out = torch.cat((out, tok), dim=-1)
        return out[..., prompt.shape[-1]:]
