"""torch.library custom ops over the C ABI of libnsa_hip.so, and the functional entry points
that mirror the reference's operator interface.

`native_sparse_attend` keeps the signature of
native_sparse_attention_pytorch/triton_native_sparse_attention.py:1938-1950 (argument names,
meaning, asserts); the op runs hand-written gfx950 kernels and nothing else - CPU tensors or a
missing library raise.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch
from torch import Tensor

from . import _lib

_BF16 = torch.bfloat16


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Tensor | None) -> int:
    return 0 if t is None else t.data_ptr()


def _rows_ok(t: Tensor) -> bool:
    return t.stride(-1) == 1 and all(s % 8 == 0 for s in t.stride()[:-1]) and t.data_ptr() % 16 == 0


def _prep(t: Tensor) -> Tensor:
    """bf16 with unit stride on the head dimension and 16-byte aligned rows (a view when it
    already is: the qkv projection's 'b n (h d) -> b h n d' view qualifies)."""
    if t.dtype != _BF16:
        raise RuntimeError(f"HIP kernels take bfloat16 tensors, got {t.dtype}")
    if not t.is_cuda:
        raise RuntimeError("HIP kernels need device tensors; there is no CPU fallback")
    return t if _rows_ok(t) else t.contiguous()


def _kernel_dim(d: int) -> int:
    """The kernels are compiled for 64 and 128 features per head; other head dimensions are zero-padded up to the next
    of the two by the wrappers below (zero features change neither the logits nor the outputs' first d features; the
    softmax scale stays that of the original dimension)."""
    if d > 128:
        raise RuntimeError(f"dim_head {d}: the HIP kernels hold at most 128 features per head")
    return 64 if d <= 64 else 128


def _pad_dim(t: Tensor, D: int) -> Tensor:
    return t if t.shape[-1] == D else torch.nn.functional.pad(t, (0, D - t.shape[-1]))


def _pad_groups(q: Tensor, hk: int):
    """The attention kernels lay the G query heads of a kv head side by side in a 32-row tile, so G must be a power of
    two.  Any other group size is padded with zero query heads (they attend uniformly, are sliced away again and get a
    zero upstream gradient, so they add nothing to dk / dv).  Returns (q', G, G')."""
    b, hq, n, d = q.shape
    g = hq // hk
    gp = 1 << max(g - 1, 0).bit_length()
    if gp == g:
        return q, g, g
    qp = torch.nn.functional.pad(q.reshape(b, hk, g, n, d), (0, 0, 0, 0, 0, gp - g)).reshape(b, hk * gp, n, d)
    return qp, g, gp


def _unpad_groups(t: Tensor, hk: int, g: int, gp: int) -> Tensor:
    """'b (hk G') n ...' -> 'b (hk G) n ...'"""
    if g == gp:
        return t
    b = t.shape[0]
    return t.reshape(b, hk, gp, *t.shape[2:])[:, :, :g].reshape(b, hk * g, *t.shape[2:])


def _select_desc(q, k, v, o, num_sel, block, causal, scale, idx_is_int64) -> _lib.SelectDesc:
    b, hq, n, d = q.shape
    hk = k.shape[1]
    dsc = _lib.SelectDesc()
    dsc.batch, dsc.kv_heads, dsc.group, dsc.seq = b, hk, hq // hk, n
    dsc.num_sel, dsc.block, dsc.dim_head, dsc.causal = num_sel, block, d, int(causal)
    dsc.idx_is_int64 = int(idx_is_int64)
    dsc.scale = scale
    for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("o_stride", o)):
        getattr(dsc, name)[:] = list(t.stride()[:3])
    return dsc


def _ws_sizes(dsc) -> tuple[int, int, int]:
    a, f, w = C.c_size_t(), C.c_size_t(), C.c_size_t()
    _lib.check(_lib.lib().nsa_select_workspace_bytes(C.byref(dsc), C.byref(a), C.byref(f), C.byref(w)), "nsa_select_workspace_bytes")
    return a.value, f.value, w.value


# A registered operator call costs about 70 us of host time here (dispatcher, schema checks, autograd wrapper), an
# autograd.Function call a fraction of that; at small shapes a layer's step is bound by exactly that cost.  Outside a
# compiler trace the attention operators therefore run as plain autograd.Functions around the same Python bodies; the
# torch.library registrations (with their fake and autograd rules) serve traced callers.
def _direct(op):
    """The Python body of a registered operator, unless a compiler is tracing (then the operator itself)."""
    return op if torch.compiler.is_compiling() else op._init_fn


def _eager_function(op, setup, backward):
    raw = op._init_fn

    class Fn(torch.autograd.Function):
        @staticmethod
        def forward(ctx, *args):
            out = raw(*args)
            setup(ctx, args, out)
            return out

        @staticmethod
        def backward(ctx, *grads):
            return backward(ctx, *grads)

    Fn.__name__ = Fn.__qualname__ = "Eager_" + getattr(op, "_name", "op")

    def call(*args):
        if torch.compiler.is_compiling():
            return op(*args)
        if not torch.is_grad_enabled() or not any(isinstance(a, Tensor) and a.requires_grad for a in args):
            return raw(*args)
        return Fn.apply(*args)
    return call


# ------------------------------------------------------------------------------- selection

@torch.library.custom_op("nsa_amd::select_fwd", mutates_args=())
def select_fwd(q: Tensor, k: Tensor, v: Tensor, idx: Tensor, fmask: Tensor, sel_scale: Optional[Tensor], block: int, causal: bool,
               scale: float) -> tuple[Tensor, Tensor, Tensor]:
    # sel_scale only takes part in the backward (its value is 1 by contract, TRI.py:1861)
    q, k, v = _prep(q), _prep(k), _prep(v)
    b, hq, n, d = q.shape
    idx = idx.contiguous()
    fm = fmask.contiguous().view(torch.uint8) if fmask.dtype == torch.bool else fmask.contiguous().to(torch.uint8)
    if idx.dtype not in (torch.int64, torch.int32):
        raise RuntimeError("selected_block_indices must be int64 or int32")
    hk = k.shape[1]
    if k.shape != (b, hk, n, d) or v.shape != k.shape or hq % hk:
        raise RuntimeError(f"q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}: expected 'b hq n d' and 'b hk n d' with hk dividing hq")
    if idx.dim() != 4 or idx.shape[:3] != (b, hk, n) or fm.shape != idx.shape or not idx.is_cuda or not fm.is_cuda:
        raise RuntimeError(f"selected_block_indices {tuple(idx.shape)} / fmask {tuple(fm.shape)}: expected device tensors 'b hk n S' with hk = {hk}")
    out = torch.empty((b, hq, n, d), dtype=_BF16, device=q.device)
    lse = torch.empty((b, hq, n), dtype=torch.float32, device=q.device)
    dsc = _select_desc(q, k, v, out, idx.shape[-1], block, causal, scale, idx.dtype == torch.int64)
    ib, fb, _ = _ws_sizes(dsc)
    index_ws = torch.empty(ib, dtype=torch.uint8, device=q.device)
    fwd_ws = torch.empty(fb, dtype=torch.uint8, device=q.device)
    L = _lib.lib()
    st = _stream()
    _lib.check(L.nsa_select_build_index(C.byref(dsc), _ptr(idx), _ptr(fm), _ptr(index_ws), ib, st), "nsa_select_build_index")
    _lib.check(L.nsa_select_fwd(C.byref(dsc), _ptr(q), _ptr(k), _ptr(v), _ptr(idx), _ptr(fm), _ptr(index_ws), _ptr(fwd_ws), fb,
                                _ptr(out), _ptr(lse), st), "nsa_select_fwd")
    return out, lse, index_ws


@select_fwd.register_fake
def _(q, k, v, idx, fmask, sel_scale, block, causal, scale):
    b, hq, n, d = q.shape
    return (q.new_empty((b, hq, n, d)), q.new_empty((b, hq, n), dtype=torch.float32), q.new_empty((1,), dtype=torch.uint8))


@torch.library.custom_op("nsa_amd::select_bwd", mutates_args=())
def select_bwd(q: Tensor, k: Tensor, v: Tensor, out: Tensor, dout: Tensor, lse: Tensor, idx: Tensor, fmask: Tensor,
               index_ws: Tensor, block: int, causal: bool, scale: float, want_sel_grads: bool,
               dlse: Optional[Tensor] = None) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    q, k, v = _prep(q), _prep(k), _prep(v)
    if dlse is not None:
        dlse = dlse.to(torch.float32).contiguous()
    out = out.contiguous()
    dout = dout.contiguous()
    if dout.dtype != _BF16:
        dout = dout.to(_BF16)
    idx = idx.contiguous()
    fm = fmask.contiguous().view(torch.uint8) if fmask.dtype == torch.bool else fmask.contiguous().to(torch.uint8)
    b, hq, n, d = q.shape
    hk = k.shape[1]
    dq = torch.empty((b, hq, n, d), dtype=_BF16, device=q.device)
    dk = torch.empty((b, hk, n, d), dtype=_BF16, device=q.device)
    dv = torch.empty((b, hk, n, d), dtype=_BF16, device=q.device)
    dsc = _select_desc(q, k, v, out, idx.shape[-1], block, causal, scale, idx.dtype == torch.int64)
    ib, _, wb = _ws_sizes(dsc)
    if index_ws.numel() < ib:
        raise RuntimeError("inverse index workspace does not belong to these shapes")
    bwd_ws = torch.empty(wb, dtype=torch.uint8, device=q.device)
    dsel = torch.empty(idx.shape if want_sel_grads else (0,), dtype=torch.float32, device=q.device)
    _lib.check(_lib.lib().nsa_select_bwd(C.byref(dsc), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(dout), _ptr(dlse), _ptr(lse), _ptr(idx), _ptr(fm),
                                         _ptr(index_ws), _ptr(bwd_ws), wb, _ptr(dq), _ptr(dk), _ptr(dv),
                                         _ptr(dsel) if want_sel_grads else 0, _stream()), "nsa_select_bwd")
    return dq, dk, dv, dsel


@select_bwd.register_fake
def _(q, k, v, out, dout, lse, idx, fmask, index_ws, block, causal, scale, want_sel_grads, dlse=None):
    return (torch.empty_like(q), torch.empty_like(k), torch.empty_like(v),
            q.new_empty(idx.shape if want_sel_grads else (0,), dtype=torch.float32))


def _select_setup(ctx, inputs, output):
    q, k, v, idx, fmask, sel_scale, block, causal, scale = inputs
    out, lse, index_ws = output
    ctx.save_for_backward(q, k, v, out, lse, idx, fmask, index_ws)
    ctx.args = (block, causal, scale, sel_scale is not None and sel_scale.requires_grad, None if sel_scale is None else sel_scale.dtype)
    ctx.set_materialize_grads(False)          # no zero tensors for the unused gradients of lse and the index workspace


def _select_backward(ctx, dout, dlse, dws):
    q, k, v, out, lse, idx, fmask, index_ws = ctx.saved_tensors
    block, causal, scale, want, sdtype = ctx.args
    if dout is None and dlse is None:
        return (None,) * 9
    if dout is None:
        dout = torch.zeros_like(out)
    dq, dk, dv, dsel = _direct(select_bwd)(q, k, v, out, dout, lse, idx, fmask, index_ws, block, causal, scale, want, dlse)
    return dq, dk, dv, None, None, (dsel.to(sdtype) if want else None), None, None, None


select_fwd.register_autograd(_select_backward, setup_context=_select_setup)
_select_fwd = _eager_function(select_fwd, _select_setup, _select_backward)


def _split_blocks(idx: Tensor, fmask: Tensor, sel_scale: Tensor | None, block: int, n: int, causal: bool):
    """The selection kernels hold a block in one or two 32-key register tiles (<= 64 keys).  A larger block is handed to
    them as m equal sub-blocks: slot s naming block j becomes the m slots 's*m + r' naming sub-blocks 'j*m + r'; under the
    causal own-block rule the sub-blocks of the query's own block that lie before the query's own sub-block are fully
    visible and become m - 1 further slots.  The softmax over the concatenated keys is the same; a gate on slot s reaches
    the kernel once per sub-block, so its gradient comes back summed.  Returns (idx, fmask, sel_scale, sub-block size)."""
    m = -(-block // 64)
    while block % m:
        m += 1
    if m == 1:
        return idx, fmask, sel_scale, block
    sub = block // m
    r = torch.arange(m, device=idx.device)
    idx_k = (idx.long()[..., None] * m + r).flatten(-2)
    fm_k = fmask.bool()[..., None].expand(*fmask.shape, m).flatten(-2)
    sc_k = None if sel_scale is None else sel_scale[..., None].expand(*sel_scale.shape, m).flatten(-2)
    if causal:
        pos = torch.arange(n, device=idx.device)
        own_idx = ((pos // block)[:, None] * m + r[None, :m - 1]).expand(*idx.shape[:2], n, m - 1)
        own_live = (r[None, :m - 1] < ((pos % block) // sub)[:, None]).expand(*idx.shape[:2], n, m - 1)
        idx_k, fm_k = torch.cat((idx_k, own_idx), dim=-1), torch.cat((fm_k, own_live), dim=-1)
        if sc_k is not None:
            sc_k = torch.cat((sc_k, sc_k.new_ones(*idx.shape[:3], m - 1)), dim=-1)
    return idx_k.contiguous(), fm_k.contiguous(), sc_k, sub


def _dead_rows_uniform(out: Tensor, fv: Tensor, selected_block_indices: Tensor, fmask: Tensor, block_size: int, q_heads: int, d: int) -> Tensor:
    """A query whose slots are all dead attends nothing in the kernels.  The reference's torch path (NSA.py:809-815)
    fills every logit of such a row with the same value, i.e. it attends uniformly over the keys of the (dead) slots'
    blocks, zero padding included; reproduce that corner with a few elementwise ops (no sync, differentiable in v)."""
    b, hs, n, S = selected_block_indices.shape
    hk2 = fv.shape[1]
    W = (n + block_size - 1) // block_size
    vpad = torch.nn.functional.pad(fv, (0, 0, 0, W * block_size - n)).reshape(b, hk2, W, block_size, d)
    vmean = vpad.float().mean(dim=3)                                                  # [b,hk,W,d]
    gi = selected_block_indices.long().clamp(0, W - 1).reshape(b, hs, n * S, 1).expand(-1, -1, -1, d)
    avg = vmean.gather(2, gi).reshape(b, hs, n, S, d).mean(dim=3)                     # [b,hk,n,d]
    dead = ~fmask.bool().any(dim=-1)                                                  # [b,hk,n]
    g = q_heads // hs
    return torch.where(dead.repeat_interleave(g, dim=1)[..., None], avg.repeat_interleave(g, dim=1).to(out.dtype), out)


_MAX_GRID_BH = 65535      # batch * kv heads of one launch (a grid dimension)
_MAX_SLOTS = 62           # slots of one call of the selection kernels (a query's live slots are a 64-bit mask, one bit the own block)


def _batch_pieces(b: int, hk: int):
    """Batch ranges whose batch * kv heads fit one launch (None: the whole batch does)."""
    if b * hk <= _MAX_GRID_BH:
        return None
    if hk > _MAX_GRID_BH:
        raise RuntimeError(f"{hk} kv heads: more than one launch can address")
    step = _MAX_GRID_BH // hk
    return [(lo, min(b, lo + step)) for lo in range(0, b, step)]


def _select_core(q: Tensor, k: Tensor, v: Tensor, idx: Tensor, fm: Tensor, sc: Tensor | None, block: int, causal: bool, scale: float):
    """select_fwd on any batch size and any number of slots: (out, lse).  A batch too large for one launch is cut along the
    batch axis; more than 62 slots are cut into groups whose results are merged by their log-sum-exp,
    out = sum_i exp(lse_i - L) out_i with L = logsumexp_i(lse_i) - the softmax over the union of the groups' keys - with the
    own block in the first group only (gradients flow through the merge: the selection backward takes d_lse)."""
    pieces = _batch_pieces(q.shape[0], k.shape[1])
    if pieces is not None:
        outs = [_select_core(q[lo:hi], k[lo:hi], v[lo:hi], idx[lo:hi], fm[lo:hi], None if sc is None else sc[lo:hi], block, causal, scale)
                for lo, hi in pieces]
        return torch.cat([o for o, _ in outs], dim=0), torch.cat([l for _, l in outs], dim=0)
    S = idx.shape[-1]
    if S <= _MAX_SLOTS:
        out, lse, _ = _select_fwd(q, k, v, idx, fm, sc, block, causal, scale)
        return out, lse
    outs, lses = [], []
    for g0 in range(0, S, _MAX_SLOTS):
        sl = slice(g0, min(S, g0 + _MAX_SLOTS))
        o, l, _ = _select_fwd(q, k, v, idx[..., sl].contiguous(), fm[..., sl].contiguous(), None if sc is None else sc[..., sl].contiguous(),
                             block, causal and g0 == 0, scale)
        outs.append(o.float())
        lses.append(l)
    L = torch.logsumexp(torch.stack(lses), dim=0)
    Ls = torch.where(torch.isfinite(L), L, torch.zeros_like(L))        # rows that attend nothing: every weight exp(-inf - 0) = 0
    out = sum(torch.exp(l - Ls)[..., None] * o for o, l in zip(outs, lses))
    return out.to(q.dtype), L


def native_sparse_attend(fq: Tensor, fk: Tensor, fv: Tensor, block_size: int, selected_block_indices: Tensor, fmask: Tensor,
                         sel_scale: Tensor | None = None, include_block_causal: bool = True, return_lse: bool = False,
                         block_dk_dv_use_dot=None, return_sliding_window_out: bool = False):
    """Drop-in for native_sparse_attend (TRI.py:1938-1987): fq [b,Hq,n,d], fk/fv [b,Hkv,n,d],
    selected_block_indices / fmask [b,Hkv|Hq,n,S].  Returns out [b,Hq,n,d] in fq's dtype and,
    on request, lse [b,Hq,n] (fp32).  Inputs are computed in bf16 (the reference computes in
    fp16, TRI.py:1845).  `sel_scale` must be all ones (straight-through gates, as the reference
    asserts at TRI.py:1861 - not re-checked here to avoid a device sync); it receives the gradient
    TRI.py:1061-1080 computes.  `block_dk_dv_use_dot` is accepted and ignored (a Triton tuning
    switch).  With `return_sliding_window_out` the outputs become pairs `(out, sliding_out)` / `(lse, sliding_lse)`
    as in the reference (TRI.py:1975-1985)."""
    q_heads, kv_heads, sel_heads = fq.shape[1], fk.shape[1], selected_block_indices.shape[1]
    assert q_heads % kv_heads == 0
    assert sel_heads in (q_heads, kv_heads)
    assert block_size >= 1
    dtype = fq.dtype
    d_head = fq.shape[-1]
    scale = d_head ** -0.5
    D = _kernel_dim(d_head)
    fv_given = fv
    fq, fk, fv = _pad_dim(fq.to(_BF16), D), _pad_dim(fk.to(_BF16), D), _pad_dim(fv.to(_BF16), D)
    sliding_out = sliding_lse = None
    if return_sliding_window_out:
        # the reference's second output (TRI.py:195-277 with SLIDING): causal attention over the last block_size + 1 keys,
        # 0 <= i - j <= block_size (test_triton_nsa.py:45-51); here it is the sliding-window kernel with that window
        qp, g0, gp0 = _pad_groups(fq.to(_BF16), kv_heads)
        sliding_out, sliding_lse, _ = dense_fwd(qp, fk, fv, 0, True, int(block_size), 1, 0, 0, 1, True, float(scale))
        sliding_out = _unpad_groups(sliding_out, kv_heads, g0, gp0)[..., :d_head].to(dtype)
        sliding_lse = _unpad_groups(sliding_lse, kv_heads, g0, gp0)
    if kv_heads != sel_heads:                         # per-query-head selection: TRI.py:1961-1962
        g = q_heads // kv_heads
        fk, fv = fk.repeat_interleave(g, dim=1), fv.repeat_interleave(g, dim=1)
    n = fq.shape[2]
    idx_in, fm_in, sc_in = selected_block_indices, fmask, sel_scale
    if block_size > 64 and n % block_size:
        # Sub-blocks that lie wholly past the sequence end would drop out of the kernel's block grid, while the reference
        # counts a selected block's zero padding (logit 0, value 0: NSA.py:744-752).  Pad to whole blocks first, as it does.
        extra = block_size - n % block_size
        padn = lambda t, value=0: torch.nn.functional.pad(t, (0, 0, 0, extra), value=value)
        fq, fk, fv = padn(fq), padn(fk), padn(fv)
        idx_in, fm_in = padn(idx_in), padn(fm_in.bool(), False)
        sc_in = None if sc_in is None else padn(sc_in, 1.0)
    qp, g0, gp0 = _pad_groups(fq, fk.shape[1])
    idx_k, fm_k, sc_k, block_k = _split_blocks(idx_in, fm_in, sc_in, int(block_size), fq.shape[2], bool(include_block_causal))
    out, lse = _select_core(qp, fk, fv, idx_k, fm_k, sc_k, block_k, bool(include_block_causal), float(scale))
    out, lse = _unpad_groups(out, fk.shape[1], g0, gp0)[:, :, :n, :d_head], _unpad_groups(lse, fk.shape[1], g0, gp0)[:, :, :n]
    fv = fv_given if kv_heads == sel_heads else fv_given.repeat_interleave(q_heads // kv_heads, dim=1)
    if not include_block_causal and selected_block_indices.shape[-1] > 0:
        out = _dead_rows_uniform(out, fv, selected_block_indices, fmask, block_size, q_heads, d_head)
    out = out.to(dtype)
    if return_sliding_window_out:
        out, lse = (out, sliding_out), (lse, sliding_lse)
    return (out, lse) if return_lse else out


# ----------------------------------------------------- sliding / compressed (interval masks)

def _dense_desc(q, k, v, o, do, mode, causal, window, stride, num_mem, pool, sel_block, share, scale) -> _lib.DenseDesc:
    b, hq, n, d = q.shape
    hk = k.shape[1]
    dsc = _lib.DenseDesc()
    dsc.batch, dsc.kv_heads, dsc.group, dsc.seq = b, hk, hq // hk, n
    dsc.num_keys, dsc.num_mem, dsc.dim_head = k.shape[2] - num_mem, num_mem, d
    dsc.mode, dsc.causal, dsc.window, dsc.stride = mode, int(causal), window, stride
    dsc.pool, dsc.sel_block, dsc.share, dsc.scale = int(pool), sel_block, int(share), scale
    for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v), ("o_stride", o), ("do_stride", do)):
        getattr(dsc, name)[:] = list(t.stride()[:3])
    return dsc


@torch.library.custom_op("nsa_amd::dense_fwd", mutates_args=())
def dense_fwd(q: Tensor, k: Tensor, v: Tensor, mode: int, causal: bool, window: int, stride: int, num_mem: int,
              pool: int, sel_block: int, share: bool, scale: float) -> tuple[Tensor, Tensor, Tensor]:
    """pool: 0 no importance logits, 1 logits with -inf wherever a block cannot be selected, 2 (causal) logits defined only
    below column i // sel_block of row i, the rest unwritten (for `importance_topk(..., prefix=...)`)."""
    q, k, v = _prep(q), _prep(k), _prep(v)
    b, hq, n, d = q.shape
    hk = k.shape[1]
    if k.dim() != 4 or k.shape[0] != b or k.shape[3] != d or v.shape != k.shape or hq % hk or k.shape[2] < num_mem:
        raise RuntimeError(f"q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}: expected 'b hq n d' and 'b hk keys d' with hk dividing hq")
    out = torch.empty((b, hq, n, d), dtype=_BF16, device=q.device)
    lse = torch.empty((b, hq, n), dtype=torch.float32, device=q.device)
    nb = 0
    if pool:
        npf = sel_block // stride
        nb = (k.shape[2] - num_mem) // npf
    pool = int(pool) if nb > 0 else 0
    pooled = torch.empty((b, hk if share else hq, n, nb), dtype=torch.float32, device=q.device)
    dsc = _dense_desc(q, k, v, out, out, mode, causal, window, stride, num_mem, pool, sel_block, share, scale)
    _lib.check(_lib.lib().nsa_dense_fwd(C.byref(dsc), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), _ptr(pooled) if pool else 0, _stream()),
               "nsa_dense_fwd")
    return out, lse, pooled


@dense_fwd.register_fake
def _(q, k, v, mode, causal, window, stride, num_mem, pool, sel_block, share, scale):
    b, hq, n, d = q.shape
    nb = ((k.shape[2] - num_mem) // (sel_block // stride)) if pool else 0
    return (q.new_empty((b, hq, n, d)), q.new_empty((b, hq, n), dtype=torch.float32),
            q.new_empty((b, k.shape[1] if share else hq, n, nb), dtype=torch.float32))


@torch.library.custom_op("nsa_amd::dense_bwd", mutates_args=())
def dense_bwd(q: Tensor, k: Tensor, v: Tensor, out: Tensor, dout: Tensor, lse: Tensor, mode: int, causal: bool, window: int,
              stride: int, num_mem: int, scale: float, dkv_fp32: bool = False) -> tuple[Tensor, Tensor, Tensor]:
    q, k, v, out = _prep(q), _prep(k), _prep(v), _prep(out)
    dout = _prep(dout if dout.dtype == _BF16 else dout.to(_BF16))
    b, hq, n, d = q.shape
    hk, nk = k.shape[1], k.shape[2]
    dq = torch.empty((b, hq, n, d), dtype=_BF16, device=q.device)
    kv_dtype = torch.float32 if dkv_fp32 else _BF16
    dk = torch.empty((b, hk, nk, d), dtype=kv_dtype, device=q.device)
    dv = torch.empty((b, hk, nk, d), dtype=kv_dtype, device=q.device)
    dsc = _dense_desc(q, k, v, out, dout, mode, causal, window, stride, num_mem, False, 1, True, scale)
    dsc.dkv_fp32 = int(dkv_fp32)
    wb = C.c_size_t()
    L = _lib.lib()
    _lib.check(L.nsa_dense_workspace_bytes(C.byref(dsc), C.byref(wb)), "nsa_dense_workspace_bytes")
    ws = torch.empty(wb.value, dtype=torch.uint8, device=q.device)
    _lib.check(L.nsa_dense_bwd(C.byref(dsc), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(dout), _ptr(lse), _ptr(ws), wb.value,
                               _ptr(dq), _ptr(dk), _ptr(dv), _stream()), "nsa_dense_bwd")
    return dq, dk, dv


@dense_bwd.register_fake
def _(q, k, v, out, dout, lse, mode, causal, window, stride, num_mem, scale, dkv_fp32=False):
    kv_dtype = torch.float32 if dkv_fp32 else k.dtype
    return torch.empty_like(q), torch.empty_like(k, dtype=kv_dtype), torch.empty_like(v, dtype=kv_dtype)


def _dense_setup(ctx, inputs, output):
    q, k, v, mode, causal, window, stride, num_mem, pool, sel_block, share, scale = inputs
    out, lse, _ = output
    ctx.save_for_backward(q, k, v, out, lse)
    ctx.args = (mode, causal, window, stride, num_mem, scale, sel_block, share)
    ctx.set_materialize_grads(False)


def _importance_backward(q, ck, dpooled, num_mem, stride, sel_block, share, scale):
    """Gradient of the importance logits (NSA.py:652-680: mean of the scaled logits over a fine
    block's npf compressed keys and, if shared, the group's heads) with respect to q and ck.  The
    logits are linear in both, so this is two small dense GEMMs per (batch, kv head); entries that
    were -inf carry zero gradient by construction of the softmax that follows."""
    b, hq, n, d = q.shape
    hk = ck.shape[1]
    g = hq // hk
    nb = dpooled.shape[-1]
    npf = sel_block // stride
    dp = torch.nan_to_num(dpooled.float(), nan=0.0, posinf=0.0, neginf=0.0)
    ckb = ck[:, :, num_mem:num_mem + nb * npf].float().reshape(b, hk, nb, npf, d).sum(dim=3)       # [b,hk,nb,d]
    qf = q.float()
    if share:
        c = scale / (g * npf)
        dq = (c * torch.matmul(dp, ckb)).repeat_interleave(g, dim=1)                                # every head of the group
        dckb = c * torch.matmul(dp.transpose(-1, -2), qf.reshape(b, hk, g, n, d).sum(dim=2))         # [b,hk,nb,d]
    else:
        c = scale / npf
        dq = c * torch.matmul(dp, ckb.repeat_interleave(g, dim=1))
        dckb = c * torch.matmul(dp.transpose(-1, -2), qf).reshape(b, hk, g, nb, d).sum(dim=2)
    dck = torch.zeros_like(ck, dtype=torch.float32)
    dck[:, :, num_mem:num_mem + nb * npf] = dckb.repeat_interleave(npf, dim=2)
    return dq, dck


def _dense_backward(ctx, dout, dlse, dpooled):
    q, k, v, out, lse = ctx.saved_tensors
    mode, causal, window, stride, num_mem, scale, sel_block, share = ctx.args
    dq = dk = dv = None
    if dout is not None:
        # the compressed keys are few and every one of their gradients is summed over all windows into the compression
        # network's parameters: they leave the kernel as fp32 and are rounded to the keys' dtype once, after the
        # importance term has been added
        dq, dk, dv = _direct(dense_bwd)(q, k, v, out, dout, lse, mode, causal, window, stride, num_mem, scale,
                                        mode == 1 and dpooled is not None and dpooled.numel() > 0)
    if dpooled is not None and dpooled.numel() > 0:
        dq2, dk2 = _importance_backward(q, k, dpooled, num_mem, stride, sel_block, share, scale)
        dq = dq2.to(q.dtype) if dq is None else (dq.float() + dq2).to(q.dtype)
        dk = dk2 if dk is None else dk.float() + dk2
    if dk is not None:
        dk, dv = dk.to(k.dtype), (dv.to(v.dtype) if dv is not None else None)
    return (dq, dk, dv) + (None,) * 9


dense_fwd.register_autograd(_dense_backward, setup_context=_dense_setup)
_dense_fwd = _eager_function(dense_fwd, _dense_setup, _dense_backward)


def sliding_attend(q: Tensor, k: Tensor, v: Tensor, window_size: int, causal: bool = True) -> Tensor:
    """Sliding-window branch: what `self.sliding_window(sq, sk, sv)` computes at NSA.py:841-850
    (LocalAttention with exact window, autopad) without materialising the repeated k/v:
    q [b,Hq,n,d], k/v [b,Hkv,n,d]; query i sees 0 <= i-j <= window_size (causal) or |i-j| <= it."""
    pieces = _batch_pieces(q.shape[0], k.shape[1])
    if pieces is not None:
        return torch.cat([sliding_attend(q[lo:hi], k[lo:hi], v[lo:hi], window_size, causal) for lo, hi in pieces], dim=0)
    d = q.shape[-1]
    D = _kernel_dim(d)
    qp, g, gp = _pad_groups(_pad_dim(q, D), k.shape[1])
    out, _, _ = _dense_fwd(qp, _pad_dim(k, D), _pad_dim(v, D), 0, bool(causal), int(window_size), 1, 0, 0, 1, True, float(d ** -0.5))
    return _unpad_groups(out, k.shape[1], g, gp)[..., :d]


def compress_attend(q: Tensor, ck: Tensor, cv: Tensor, num_mem: int, stride: int, causal: bool,
                    sel_block: int | None = None, share: bool = True, prefix_only: bool = False):
    """Compressed branch: attend(q, [mem; ck], [mem; cv], cmask, return_sim=True) of NSA.py:621-639.
    Returns (out, importance_logits) where importance_logits [b, Hkv|Hq, n, nb] are the block
    importance logits of NSA.py:652-691 before the softmax (None if sel_block is None or no full
    fine block exists): the logits matrix itself is never written to memory.
    With `prefix_only` the result is (out, importance_logits, prefix): if `prefix` is not None it is (n, sel_block) and row i
    of the logits is defined only below column i // sel_block - what a causal query can select from; the rest (all -inf
    otherwise) was not written and must not be read: pass `prefix` on to `importance_topk`.  Only for logits nothing else
    reads (no gradient through them)."""
    pieces = _batch_pieces(q.shape[0], ck.shape[1])
    if pieces is not None:
        parts = [compress_attend(q[lo:hi], ck[lo:hi], cv[lo:hi], num_mem, stride, causal, sel_block, share, prefix_only) for lo, hi in pieces]
        cat = lambda ts: None if ts[0] is None else torch.cat(ts, dim=0)
        res = (cat([p_[0] for p_ in parts]), cat([p_[1] for p_ in parts]))
        return res + (parts[0][2],) if prefix_only else res
    pool = sel_block is not None
    d = q.shape[-1]
    scale = float(d ** -0.5)
    D = _kernel_dim(d)
    npf = int(sel_block) // int(stride) if pool else 1
    hk = ck.shape[1]
    q, g, gp = _pad_groups(_pad_dim(q, D), hk)
    ck, cv = _pad_dim(ck, D), _pad_dim(cv, D)

    def logits_of(pooled):
        # zero padding heads add nothing to a group's sum: the kernel's mean over G' heads becomes the mean over G;
        # per-head logits of the padding heads are dropped
        if g == gp:
            return pooled
        return pooled * (gp / g) if share else _unpad_groups(pooled, hk, g, gp)
    if pool and (npf > 32 or npf & (npf - 1)):
        # The kernel pools groups of 1, 2, 4 .. 32 compressed keys.  Other ratios (a selection block of 20 over stride 4, as in
        # the reference's own inference test) take the per-key logits from the kernel (a "block" of one key: head mean and
        # visibility as usual) and finish NSA.py:676-689 with three elementwise ops: mean over the block's keys (-inf as
        # soon as one key is invisible), own block masked.
        out, _, per_key = _dense_fwd(q, ck, cv, 1, bool(causal), 0, int(stride), int(num_mem), 1, int(stride), bool(share), scale)
        out = _unpad_groups(out, hk, g, gp)[..., :d]
        n, nb = q.shape[2], per_key.shape[-1] // npf
        if nb == 0:
            return (out, None, None) if prefix_only else (out, None)
        imp = logits_of(per_key)[..., :nb * npf].unflatten(-1, (nb, npf)).mean(dim=-1)
        own = (torch.arange(n, device=q.device) // int(sel_block))[:, None] == torch.arange(nb, device=q.device)[None, :]
        imp = imp.masked_fill(own, float("-inf"))
        return (out, imp, None) if prefix_only else (out, imp)
    use_prefix = bool(prefix_only and pool and causal and g == gp)
    out, _, pooled = _dense_fwd(q, ck, cv, 1, bool(causal), 0, int(stride), int(num_mem), (2 if use_prefix else 1) if pool else 0,
                                int(sel_block or stride), bool(share), scale)
    out = _unpad_groups(out, hk, g, gp)[..., :d]
    imp = logits_of(pooled) if pool and pooled.shape[-1] > 0 else None
    if not prefix_only:
        return out, imp
    return out, imp, ((q.shape[2], int(sel_block)) if use_prefix and imp is not None else None)


@torch.library.custom_op("nsa_amd::compress_topk_fwd", mutates_args=())
def compress_topk_fwd(q: Tensor, k: Tensor, v: Tensor, causal: bool, stride: int, num_mem: int, sel_block: int, num_sel: int,
                      scale: float) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    """Compressed attention whose kernel also selects the blocks (nsa_compress_topk_fwd): (out, lse, idx int32, fmask uint8)."""
    q, k, v = _prep(q), _prep(k), _prep(v)
    b, hq, n, d = q.shape
    hk = k.shape[1]
    if k.dim() != 4 or k.shape[0] != b or k.shape[3] != d or v.shape != k.shape or hq % hk or k.shape[2] < num_mem:
        raise RuntimeError(f"q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}: expected 'b hq n d' and 'b hk keys d' with hk dividing hq")
    out = torch.empty((b, hq, n, d), dtype=_BF16, device=q.device)
    lse = torch.empty((b, hq, n), dtype=torch.float32, device=q.device)
    idx = torch.empty((b, hk, n, num_sel), dtype=torch.int32, device=q.device)
    fm = torch.empty((b, hk, n, num_sel), dtype=torch.uint8, device=q.device)
    dsc = _dense_desc(q, k, v, out, out, 1, causal, 0, stride, num_mem, 1, sel_block, True, scale)
    _lib.check(_lib.lib().nsa_compress_topk_fwd(C.byref(dsc), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), int(num_sel), _ptr(idx), _ptr(fm),
                                                _stream()), "nsa_compress_topk_fwd")
    return out, lse, idx, fm


@compress_topk_fwd.register_fake
def _(q, k, v, causal, stride, num_mem, sel_block, num_sel, scale):
    b, hq, n, d = q.shape
    hk = k.shape[1]
    return (q.new_empty((b, hq, n, d)), q.new_empty((b, hq, n), dtype=torch.float32),
            q.new_empty((b, hk, n, num_sel), dtype=torch.int32), q.new_empty((b, hk, n, num_sel), dtype=torch.uint8))


def _compress_topk_setup(ctx, inputs, output):
    q, k, v, causal, stride, num_mem, sel_block, num_sel, scale = inputs
    out, lse, _, _ = output
    ctx.save_for_backward(q, k, v, out, lse)
    ctx.args = (causal, stride, num_mem, scale)
    ctx.set_materialize_grads(False)


def _compress_topk_backward(ctx, dout, dlse, didx, dfm):
    q, k, v, out, lse = ctx.saved_tensors
    causal, stride, num_mem, scale = ctx.args
    if dout is None:
        return (None,) * 9
    dq, dk, dv = _direct(dense_bwd)(q, k, v, out, dout, lse, 1, causal, 0, stride, num_mem, scale, False)
    return (dq, dk, dv) + (None,) * 6


compress_topk_fwd.register_autograd(_compress_topk_backward, setup_context=_compress_topk_setup)
_compress_topk_fwd = _eager_function(compress_topk_fwd, _compress_topk_setup, _compress_topk_backward)


def compress_topk_supported(q: Tensor, ck: Tensor, num_mem: int, stride: int, sel_block: int, num_selected: int, share: bool) -> bool:
    """Whether `compress_attend_topk` serves these shapes (else: `compress_attend` + `importance_topk`)."""
    d = q.shape[-1]
    hk = ck.shape[1]
    g = q.shape[1] // hk
    npf = int(sel_block) // int(stride)
    nb = (ck.shape[2] - num_mem) // max(npf, 1)
    return bool(share and q.is_cuda and d <= 128 and g >= 2 and not (g & (g - 1)) and npf >= 1 and npf <= 32 and not (npf & (npf - 1))
                and int(sel_block) % int(stride) == 0 and 1 <= num_selected <= min(16, nb))


def compress_attend_topk(q: Tensor, ck: Tensor, cv: Tensor, num_mem: int, stride: int, causal: bool, sel_block: int, num_selected: int):
    """Compressed branch and block selection in one kernel: attend(q, [mem; ck], [mem; cv], cmask) of NSA.py:621-639 and, from
    its logits, the importance scores, padded softmax, top-k and slot mask of NSA.py:652-721 (selections shared by the heads of a
    group).  The importance logits are never written to memory.  Returns (out, idx int32 'b hk n k', fmask bool); `out` is
    differentiable, the selection carries no gradient (for the differentiable top-k use compress_attend + importance_topk).
    Needs compress_topk_supported(...)."""
    pieces = _batch_pieces(q.shape[0], ck.shape[1])
    if pieces is not None:
        parts = [compress_attend_topk(q[lo:hi], ck[lo:hi], cv[lo:hi], num_mem, stride, causal, sel_block, num_selected) for lo, hi in pieces]
        return tuple(torch.cat([p_[t] for p_ in parts], dim=0) for t in range(3))
    d = q.shape[-1]
    D = _kernel_dim(d)
    hk = ck.shape[1]
    q2, g, gp = _pad_groups(_pad_dim(q, D), hk)
    if g != gp:
        raise RuntimeError("compress_attend_topk: the group size must be a power of two")
    out, _, idx, fm = _compress_topk_fwd(q2, _pad_dim(ck, D), _pad_dim(cv, D), bool(causal), int(stride), int(num_mem), int(sel_block),
                                         int(num_selected), float(d ** -0.5))
    return out[..., :d], idx, fm.view(torch.bool)


# ------------------------------------------------------------------------------------ top-k

_TOPK_MAX_ROW, _TOPK_MAX_K = 2048, 64      # one call of the top-k kernel: a row in the registers of one wave, one result per lane


def _topk_large(scores: Tensor, k: int, apply_softmax: bool, prefix=None):
    """Rows longer than 2048 entries or more than 64 selections (the reference's topk, NSA.py:703-713, has no limit): the
    padded softmax over the whole row is taken first (NSA.py:693-695, elementwise torch), then the kernel selects per
    segment of 2048 columns and once more among the segments' winners, 64 at a time, taken entries struck out in between.
    The tie rule survives both steps: a segment lists equal values lower index first, and the winners of a lower segment
    stand before those of a higher one."""
    nb = scores.shape[-1]
    work = scores
    if prefix is not None:
        seq, block = prefix
        lim = (torch.arange(seq, device=scores.device) // block)[:, None]
        work = work.masked_fill(torch.arange(nb, device=scores.device)[None, :] >= lim, float("-inf"))
    if apply_softmax:
        work = torch.nn.functional.pad(work, (1, 0), value=-1e3).softmax(dim=-1)[..., 1:]
    work = work.contiguous().clone()
    segs = [(lo, min(nb, lo + _TOPK_MAX_ROW)) for lo in range(0, nb, _TOPK_MAX_ROW)]
    idx_parts, val_parts = [], []
    left = k
    while left > 0:
        kk = min(_TOPK_MAX_K, left)
        cand_v, cand_i = [], []
        for lo, hi in segs:
            ks = min(kk, hi - lo)
            i_s, v_s, _ = _topk_impl(work[..., lo:hi].contiguous(), ks, False)
            cand_v.append(v_s)
            cand_i.append(i_s.long() + lo)
        cv_, ci_ = torch.cat(cand_v, dim=-1), torch.cat(cand_i, dim=-1)
        if len(segs) > 1:
            if cv_.shape[-1] > _TOPK_MAX_ROW:
                raise RuntimeError(f"top-k over {nb} entries with k = {k}: more candidates than one merge step holds")
            pos, v_m, _ = _topk_impl(torch.nan_to_num(cv_, nan=float("inf")).contiguous(), kk, False)
            i_m = ci_.gather(-1, pos.long())
            v_m = cv_.gather(-1, pos.long())
        else:
            i_m, v_m = ci_, cv_
        idx_parts.append(i_m)
        val_parts.append(v_m)
        work.scatter_(-1, i_m, -3.0)                    # below every probability and the kernel's own markers
        left -= kk
    idx = torch.cat(idx_parts, dim=-1).to(torch.int32)
    vals = torch.cat(val_parts, dim=-1)
    fm = ((vals > 1e-10) & torch.isfinite(vals)).to(torch.uint8)
    return idx, vals, fm


def _topk_impl(scores: Tensor, k: int, apply_softmax: bool, prefix=None):
    if scores.dtype != torch.float32 or not scores.is_cuda:
        raise RuntimeError("importance scores must be fp32 device tensors")
    if scores.shape[-1] > _TOPK_MAX_ROW or k > _TOPK_MAX_K:
        if k > scores.shape[-1]:
            raise RuntimeError(f"top-k of {k} among {scores.shape[-1]} entries")
        return _topk_large(scores, int(k), bool(apply_softmax), prefix)
    scores = scores.contiguous()
    nb = scores.shape[-1]
    rows = scores.numel() // nb
    shp = (*scores.shape[:-1], k)
    idx = torch.empty(shp, dtype=torch.int32, device=scores.device)
    vals = torch.empty(shp, dtype=torch.float32, device=scores.device)
    fm = torch.empty(shp, dtype=torch.uint8, device=scores.device)
    if prefix is not None:
        seq, block = prefix
        if scores.shape[-2] != seq:
            raise RuntimeError(f"prefix {prefix}: the logits have {scores.shape[-2]} rows per sequence")
        _lib.check(_lib.lib().nsa_topk_prefix(_ptr(scores), rows, nb, k, int(apply_softmax), int(seq), int(block), _ptr(idx), _ptr(vals), _ptr(fm),
                                              _stream()), "nsa_topk_prefix")
    else:
        _lib.check(_lib.lib().nsa_topk(_ptr(scores), rows, nb, k, int(apply_softmax), _ptr(idx), _ptr(vals), _ptr(fm), _stream()), "nsa_topk")
    return idx, vals, fm


@torch.library.custom_op("nsa_amd::topk", mutates_args=())
def topk_op(scores: Tensor, k: int, apply_softmax: bool) -> tuple[Tensor, Tensor, Tensor]:
    return _topk_impl(scores, k, apply_softmax)


@topk_op.register_fake
def _(scores, k, apply_softmax):
    shp = (*scores.shape[:-1], k)
    return (scores.new_empty(shp, dtype=torch.int32), scores.new_empty(shp), scores.new_empty(shp, dtype=torch.uint8))


@torch.library.custom_op("nsa_amd::topk_prefix", mutates_args=())
def topk_prefix_op(scores: Tensor, k: int, apply_softmax: bool, seq: int, block: int) -> tuple[Tensor, Tensor, Tensor]:
    return _topk_impl(scores, k, apply_softmax, (seq, block))


@topk_prefix_op.register_fake
def _(scores, k, apply_softmax, seq, block):
    shp = (*scores.shape[:-1], k)
    return (scores.new_empty(shp, dtype=torch.int32), scores.new_empty(shp), scores.new_empty(shp, dtype=torch.uint8))


class _ImportanceTopk(torch.autograd.Function):
    """HIP top-k in the forward; the backward of `values` through the padded softmax (plain
    elementwise torch, O(rows * nb)) - only used for the differentiable top-k gates."""

    @staticmethod
    def forward(ctx, logits, k):
        idx, vals, fm = topk_op(logits, k, True)
        ctx.save_for_backward(logits, idx)
        ctx.mark_non_differentiable(idx, fm)
        return vals, idx, fm

    @staticmethod
    def backward(ctx, dvals, _didx, _dfm):
        logits, idx = ctx.saved_tensors
        padded = torch.nn.functional.pad(logits, (1, 0), value=-1e3)
        p = padded.softmax(dim=-1)[..., 1:]                     # -inf entries -> exactly 0
        dfull = torch.zeros_like(p).scatter_add_(-1, idx.long(), dvals.to(p.dtype))
        dl = p * (dfull - (p * dfull).sum(dim=-1, keepdim=True))
        return dl, None


def importance_topk(importance_logits: Tensor, num_selected: int, prefix=None):
    """softmax with the -1e3 pad column (NSA.py:693-695) + topk (NSA.py:713) + `> 1e-10` mask
    (NSA.py:721).  Returns (values fp32, indices int32, fmask bool), each [..., num_selected];
    `values` is differentiable with respect to the logits.  `prefix` = (n, sel_block) as returned by
    `compress_attend(..., prefix_only=True)`: row i is read only below column i // sel_block (no gradient)."""
    if prefix is not None:
        if torch.compiler.is_compiling():
            idx, vals, fm = topk_prefix_op(importance_logits.detach(), int(num_selected), True, int(prefix[0]), int(prefix[1]))
        else:
            idx, vals, fm = _topk_impl(importance_logits.detach(), int(num_selected), True, prefix)
        return vals, idx, fm.view(torch.bool)
    if importance_logits.requires_grad and torch.is_grad_enabled():
        vals, idx, fm = _ImportanceTopk.apply(importance_logits, int(num_selected))
    elif torch.compiler.is_compiling():
        idx, vals, fm = topk_op(importance_logits, int(num_selected), True)
    else:
        idx, vals, fm = _topk_impl(importance_logits, int(num_selected), True)     # eager inference: skip the dispatcher
    return vals, idx, fm.view(torch.bool)


# --------------------------------------------------------------------------------- gate

def _s3(t: Tensor):
    return (C.c_int64 * 3)(*t.stride()[:3])


@torch.library.custom_op("nsa_amd::gate_fwd", mutates_args=())
def gate_fwd(logits: Tensor, c: Tensor, f: Tensor, s: Tensor) -> Tensor:
    c, f, s = _prep(c), _prep(f), _prep(s)
    logits = logits.contiguous()
    if logits.dtype != _BF16:
        raise RuntimeError("gate logits must be bfloat16")
    b, h, n, d = c.shape
    out = torch.empty((b, n, h * d), dtype=_BF16, device=c.device)
    _lib.check(_lib.lib().nsa_gate_fwd(b, h, n, d, _ptr(logits), _ptr(c), _s3(c), _ptr(f), _s3(f), _ptr(s), _s3(s), _ptr(out), _stream()),
               "nsa_gate_fwd")
    return out


@gate_fwd.register_fake
def _(logits, c, f, s):
    b, h, n, d = c.shape
    return c.new_empty((b, n, h * d))


@torch.library.custom_op("nsa_amd::gate_bwd", mutates_args=())
def gate_bwd(logits: Tensor, c: Tensor, f: Tensor, s: Tensor, dout: Tensor) -> tuple[Tensor, Tensor, Tensor, Tensor]:
    c, f, s = _prep(c), _prep(f), _prep(s)
    logits = logits.contiguous()
    dout = dout.contiguous()
    if dout.dtype != _BF16:
        dout = dout.to(_BF16)
    b, h, n, d = c.shape
    dl = torch.empty_like(logits)
    dc, df, ds = (torch.empty((b, h, n, d), dtype=_BF16, device=c.device) for _ in range(3))
    _lib.check(_lib.lib().nsa_gate_bwd(b, h, n, d, _ptr(logits), _ptr(c), _s3(c), _ptr(f), _s3(f), _ptr(s), _s3(s), _ptr(dout),
                                       _ptr(dl), _ptr(dc), _ptr(df), _ptr(ds), _stream()), "nsa_gate_bwd")
    return dl, dc, df, ds


@gate_bwd.register_fake
def _(logits, c, f, s, dout):
    return torch.empty_like(logits), torch.empty_like(c), torch.empty_like(f), torch.empty_like(s)


def _gate_setup(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


def _gate_backward(ctx, dout):
    logits, c, f, s = ctx.saved_tensors
    return _direct(gate_bwd)(logits, c, f, s, dout)


gate_fwd.register_autograd(_gate_backward, setup_context=_gate_setup)
_gate_fwd = _eager_function(gate_fwd, _gate_setup, _gate_backward)


def gate_combine(logits: Tensor, compressed: Tensor, selected: Tensor, sliding: Tensor) -> Tensor:
    """sigmoid(logits) 'b n (h s) -> b h n s' weighted sum of the three branches, merged to
    'b n (h d)' (NSA.py:323-327, 854-860).  logits are the pre-sigmoid gate projection."""
    b, h, n, d = compressed.shape
    D = _kernel_dim(d)
    out = _gate_fwd(logits.to(_BF16), _pad_dim(compressed, D), _pad_dim(selected, D), _pad_dim(sliding, D))
    return out if D == d else out.reshape(b, n, h, D)[..., :d].reshape(b, n, h * d)


# ---------------------------------------------------------------------------------- rotary

@torch.library.custom_op("nsa_amd::rope", mutates_args=())
def rope_op(x: Tensor, freqs: Tensor, offset: int, inverse: bool) -> Tensor:
    x = _prep(x)
    b, h, n, d = x.shape
    freqs = freqs.detach().to(torch.float32).contiguous()
    out = torch.empty((b, h, n, d), dtype=_BF16, device=x.device)
    _lib.check(_lib.lib().nsa_rope(_ptr(x), _s3(x), b, h, n, d, _ptr(freqs), int(offset), int(inverse), _ptr(out), None, _stream()), "nsa_rope")
    return out


@rope_op.register_fake
def _(x, freqs, offset, inverse):
    return x.new_empty(x.shape)


def _rope_setup(ctx, inputs, output):
    _, freqs, offset, inverse = inputs
    ctx.save_for_backward(freqs)
    ctx.args = (offset, inverse)


def _rope_backward(ctx, dout):
    (freqs,) = ctx.saved_tensors
    offset, inverse = ctx.args
    return rope_op(dout if dout.dtype == _BF16 else dout.to(_BF16), freqs, offset, not inverse), None, None, None


rope_op.register_autograd(_rope_backward, setup_context=_rope_setup)


# q and k of a layer in one operator call: at small shapes a layer's step is bound by the host-side cost of its
# operator calls (~70 us each through torch.library), not by the kernels
@torch.library.custom_op("nsa_amd::rope_pair", mutates_args=())
def rope_pair_op(q: Tensor, k: Tensor, freqs: Tensor, offset: int, inverse: bool) -> tuple[Tensor, Tensor]:
    freqs = freqs.detach().to(torch.float32).contiguous()
    outs = []
    for x in (q, k):
        x = _prep(x)
        b, h, n, d = x.shape
        out = torch.empty((b, h, n, d), dtype=_BF16, device=x.device)
        _lib.check(_lib.lib().nsa_rope(_ptr(x), _s3(x), b, h, n, d, _ptr(freqs), int(offset), int(inverse), _ptr(out), None, _stream()), "nsa_rope")
        outs.append(out)
    return outs[0], outs[1]


@rope_pair_op.register_fake
def _(q, k, freqs, offset, inverse):
    return q.new_empty(q.shape), k.new_empty(k.shape)


def _rope_pair_setup(ctx, inputs, output):
    _, _, freqs, offset, inverse = inputs
    ctx.save_for_backward(freqs)
    ctx.args = (offset, inverse)


def _rope_pair_backward(ctx, dq, dk):
    (freqs,) = ctx.saved_tensors
    offset, inverse = ctx.args
    dq, dk = rope_pair_op(dq if dq.dtype == _BF16 else dq.to(_BF16), dk if dk.dtype == _BF16 else dk.to(_BF16), freqs, offset, not inverse)
    return dq, dk, None, None, None


rope_pair_op.register_autograd(_rope_pair_backward, setup_context=_rope_pair_setup)


def rotary_pair(q: Tensor, k: Tensor, freqs: Tensor, offset: int = 0):
    """`rotary` of the queries and the keys of a layer in one operator call."""
    d = q.shape[-1]
    D = _kernel_dim(d)
    if D == d:
        return rope_pair_op(q, k, freqs, int(offset), False)
    rq, rk = rope_pair_op(_pad_dim(q, D), _pad_dim(k, D), _pad_dim(freqs, D // 2), int(offset), False)
    return rq[..., :d], rk[..., :d]


def rotary(x: Tensor, freqs: Tensor, offset: int = 0) -> Tensor:
    """Rotary embedding of 'b h n d' queries or keys at positions offset .. offset+n-1 (NSA.py:643)."""
    d = x.shape[-1]
    D = _kernel_dim(d)
    if D == d:
        return rope_op(x, freqs, int(offset), False)
    # padded feature pairs get frequency 0: they stay zero
    return rope_op(_pad_dim(x, D), _pad_dim(freqs, D // 2), int(offset), False)[..., :d]


def rotary_into(x: Tensor, freqs: Tensor, offset: int, out: Tensor) -> None:
    """Rotate 'b h n d' `x` at positions offset.. and write the result into `out`, a strided
    'b h n d' view (a slot of a key cache, NSA.py:384-390).  Inference only (no autograd)."""
    x = _prep(x)
    b, h, n, d = x.shape
    if out.dtype != _BF16 or out.shape != x.shape or not _rows_ok(out):
        raise RuntimeError("rotary_into: `out` must be a bf16 'b h n d' view with 16-byte aligned rows")
    freqs = freqs.detach().to(torch.float32).contiguous()
    _lib.check(_lib.lib().nsa_rope(_ptr(x), _s3(x), b, h, n, d, _ptr(freqs), int(offset), 0, _ptr(out), _s3(out), _stream()), "nsa_rope")


# ---------------------------------------------------------------------------------- decode

def _decode_call(dsc, q, k, v, mem_k, mem_v, idx, fmask, logits, merge=True):
    """Runs the split-K walk; with merge the head outputs 'b hq 1 d', otherwise the workspace
    holding the partials (for decode_combine)."""
    L = _lib.lib()
    nbytes = C.c_size_t()
    _lib.check(L.nsa_decode_workspace_bytes(C.byref(dsc), C.byref(nbytes)), "nsa_decode_workspace_bytes")
    ws = torch.empty(max(nbytes.value, 16), dtype=torch.uint8, device=q.device)
    out = torch.empty((q.shape[0], q.shape[1], 1, q.shape[3]), dtype=_BF16, device=q.device) if merge else None
    _lib.check(L.nsa_decode_attend(C.byref(dsc), _ptr(q), _ptr(k), _ptr(v), _ptr(mem_k), _ptr(mem_v), _ptr(idx), _ptr(fmask),
                                   _ptr(ws), nbytes, _ptr(out), _ptr(logits), _stream()), "nsa_decode_attend")
    return out if merge else (dsc, ws)


def _decode_desc(q: Tensor, k: Tensor | None, v: Tensor | None, hk: int):
    b, hq, one, d = q.shape
    if one != 1:
        raise RuntimeError("decode attention takes one query token")
    if hq % hk:
        raise RuntimeError("query heads must be a multiple of kv heads")
    dsc = _lib.DecodeDesc()
    dsc.batch, dsc.kv_heads, dsc.group, dsc.dim_head = b, hk, hq // hk, d
    dsc.scale = d ** -0.5
    dsc.q_stride[:] = (q.stride(0), q.stride(1))
    for name, t in (("k_stride", k), ("v_stride", v)):
        if t is not None:
            if t.dtype != _BF16 or not t.is_cuda or not _rows_ok(t):
                raise RuntimeError("key / value caches must be bf16 device tensors with unit feature stride and 16-byte aligned rows")
            getattr(dsc, name)[:] = t.stride()[:3]
    return dsc


@torch.no_grad()
def decode_range_attend(q: Tensor, k: Tensor, v: Tensor, start: int, count: int, mem_k: Tensor | None = None,
                        mem_v: Tensor | None = None, return_logits: bool = False, merge: bool = True):
    """One query token 'b hq 1 d' attends keys [start, start+count) of the caches 'b hk cap d',
    preceded by the memory rows mem_k / mem_v 'hk m d' (compressed branch NSA.py:396-420; sliding
    branch NSA.py:519-530).  With return_logits also scale * q.k over the cache keys, fp32
'b hq count' (NSA.py:444).  merge=False returns a handle for decode_combine in place of
    the output."""
    q = _prep(q)
    hk = k.shape[1]
    if start < 0 or count < 0 or start + count > k.shape[2] or k.shape != v.shape:
        raise RuntimeError("decode_range_attend: key range outside the caches")
    dsc = _decode_desc(q, k if count else None, v if count else None, hk)
    dsc.mode, dsc.start, dsc.count = 0, int(start), int(count)
    m = 0
    if mem_k is not None:
        mem_k, mem_v = mem_k.to(_BF16).contiguous(), mem_v.to(_BF16).contiguous()
        m = mem_k.shape[-2]
        if mem_k.shape != (hk, m, q.shape[-1]) or mem_v.shape != mem_k.shape:
            raise RuntimeError("decode_range_attend: memory rows must be 'hk m d'")
    dsc.num_mem = m
    logits = torch.empty((q.shape[0], q.shape[1], count), dtype=torch.float32, device=q.device) if return_logits else None
    out = _decode_call(dsc, q, k if count else None, v if count else None, mem_k, mem_v, None, None, logits, merge)
    return (out, logits) if return_logits else out


@torch.no_grad()
def decode_select_attend(q: Tensor, k: Tensor, v: Tensor, kv_len: int, block: int, idx: Tensor, fmask: Tensor, merge: bool = True):
    """One query token at position kv_len-1 attends the blocks idx[..., slot] (where fmask) and
    its own block up to itself (NSA.py:446-515).  idx / fmask: 'b hk 1 S' or, for per-head
    selection, 'b hq 1 S'."""
    q = _prep(q)
    b, hq = q.shape[:2]
    hk = k.shape[1]
    if kv_len < 1 or kv_len > k.shape[2] or k.shape != v.shape:
        raise RuntimeError("decode_select_attend: kv_len outside the caches")
    if idx.shape[:3] not in ((b, hk, 1), (b, hq, 1)) or fmask.shape != idx.shape:
        raise RuntimeError("decode_select_attend: idx / fmask must be 'b hk 1 S' or 'b hq 1 S'")
    if idx.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("decode_select_attend: idx must be int32 or int64")
    dsc = _decode_desc(q, k, v, hk)
    dsc.mode, dsc.block, dsc.num_sel, dsc.kv_len = 1, int(block), idx.shape[-1], int(kv_len)
    dsc.per_head_sel = int(idx.shape[1] == hq and hq != hk)
    dsc.idx_is_int64 = int(idx.dtype == torch.int64)
    idx = idx.contiguous()
    fm = fmask.contiguous().view(torch.uint8) if fmask.dtype == torch.bool else fmask.to(torch.uint8).contiguous()
    return _decode_call(dsc, q, k, v, None, None, idx if idx.numel() else None, fm if fm.numel() else None, None, merge)


@torch.no_grad()
def decode_combine(gate_logits: Tensor, compressed, selected, sliding) -> Tensor:
    """Merges the three branches (handles from decode_*_attend(..., merge=False); None for a
    branch that contributes nothing), applies sigmoid(gate_logits 'b 1 (h 3)') and merges the
    heads: 'b 1 (h d)' (NSA.py:534-545)."""
    ref = next(h for h in (compressed, selected, sliding) if h is not None)[0]
    b, hq, d = ref.batch, ref.kv_heads * ref.group, ref.dim_head
    gl = gate_logits.to(_BF16).contiguous()
    if gl.numel() != b * hq * 3:
        raise RuntimeError("decode_combine: gate logits must be 'b 1 (h 3)'")
    out = torch.empty((b, 1, hq * d), dtype=_BF16, device=gl.device)
    args = []
    for h in (compressed, selected, sliding):
        args += [None, None] if h is None else [C.byref(h[0]), _ptr(h[1])]
    _lib.check(_lib.lib().nsa_decode_combine(*args, _ptr(gl), _ptr(out), _stream()), "nsa_decode_combine")
    return out


@torch.no_grad()
def decode_prep(q: Tensor, k: Tensor, v: Tensor, freqs: Tensor, pos: int, k_row: Tensor, v_row: Tensor,
                k_run_row: Tensor | None = None, v_run_row: Tensor | None = None) -> Tensor:
    """New token's q 'b hq 1 d', k, v 'b hk 1 d' (bf16 views are fine): returns the rotated
    queries and writes the rotated keys / the values into the cache rows k_row, v_row 'b hk 1 d'
    (NSA.py:384-393) and, when given, the un-rotated keys / values into k_run_row, v_run_row (the
    open compression window, NSA.py:377-380)."""
    q, k, v = _prep(q), _prep(k), _prep(v)
    b, hq, _, d = q.shape
    hk = k.shape[1]
    for t in (k_row, v_row, k_run_row, v_run_row):
        if t is not None and (t.dtype != _BF16 or t.shape != (b, hk, 1, d) or not _rows_ok(t)):
            raise RuntimeError("decode_prep: cache rows must be bf16 'b hk 1 d' views with 16-byte aligned rows")
    freqs = freqs.detach()
    if freqs.dtype != torch.float32 or not freqs.is_contiguous():
        freqs = freqs.to(torch.float32).contiguous()
    rq = torch.empty((b, hq, 1, d), dtype=_BF16, device=q.device)
    s2 = lambda t: (C.c_int64 * 2)(t.stride(0), t.stride(1))
    run = k_run_row is not None and v_run_row is not None
    _lib.check(_lib.lib().nsa_decode_prep(_ptr(q), s2(q), _ptr(k), s2(k), _ptr(v), s2(v), b, hq, hk, d, _ptr(freqs), int(pos), _ptr(rq),
                                          _ptr(k_row), s2(k_row), _ptr(v_row), s2(v_row),
                                          _ptr(k_run_row) if run else None, s2(k_run_row) if run else None,
                                          _ptr(v_run_row) if run else None, s2(v_run_row) if run else None, _stream()), "nsa_decode_prep")
    return rq


# ---------------------------------------------------------------------- compression windows

@torch.library.custom_op("nsa_amd::windows_fwd", mutates_args=())
def windows_fwd(x: Tensor, pos: Optional[Tensor], block: int, stride: int) -> Tensor:
    x = _prep(x)
    b, h, n, d = x.shape
    w = n // stride
    out = torch.empty((b, h, w, block, d), dtype=_BF16, device=x.device)
    if pos is not None:
        pos = pos.to(_BF16).contiguous()
        if pos.shape != (h, block, d):
            raise RuntimeError("window positions must be 'h block d'")
    if w > 0:
        _lib.check(_lib.lib().nsa_windows_fwd(_ptr(x), _s3(x), _ptr(pos), b, h, n, d, int(block), int(stride), _ptr(out), _stream()), "nsa_windows_fwd")
    return out


@windows_fwd.register_fake
def _(x, pos, block, stride):
    b, h, n, d = x.shape
    return x.new_empty((b, h, n // stride, block, d))


@torch.library.custom_op("nsa_amd::windows_bwd", mutates_args=())
def windows_bwd(dwin: Tensor, n: int, stride: int) -> Tensor:
    dwin = dwin.contiguous()
    if dwin.dtype != _BF16:
        raise RuntimeError("window gradients must be bfloat16")
    b, h, w, block, d = dwin.shape
    dx = torch.empty((b, h, n, d), dtype=_BF16, device=dwin.device)
    if w == 0:
        return dx.zero_()
    _lib.check(_lib.lib().nsa_windows_bwd(_ptr(dwin), b, h, n, d, block, int(stride), _ptr(dx), _stream()), "nsa_windows_bwd")
    return dx


@windows_bwd.register_fake
def _(dwin, n, stride):
    b, h, w, block, d = dwin.shape
    return dwin.new_empty((b, h, n, d))


def _windows_setup(ctx, inputs, output):
    x, pos, block, stride = inputs
    ctx.n, ctx.stride, ctx.has_pos = x.shape[2], stride, pos is not None
    ctx.pos_dtype = pos.dtype if pos is not None else None


def _windows_backward(ctx, dwin):
    dwin = dwin if dwin.dtype == _BF16 else dwin.to(_BF16)
    dx = windows_bwd(dwin, ctx.n, ctx.stride)
    dpos = dwin.sum(dim=(0, 2), dtype=torch.float32).to(ctx.pos_dtype) if ctx.has_pos else None
    return dx, dpos, None, None


windows_fwd.register_autograd(_windows_backward, setup_context=_windows_setup)


# keys and values of a layer in one operator call (see rope_pair_op)
@torch.library.custom_op("nsa_amd::windows_pair_fwd", mutates_args=())
def windows_pair_fwd(k: Tensor, v: Tensor, kpos: Tensor, vpos: Tensor, block: int, stride: int) -> tuple[Tensor, Tensor]:
    outs = []
    for x, pos in ((k, kpos), (v, vpos)):
        x = _prep(x)
        b, h, n, d = x.shape
        w = n // stride
        out = torch.empty((b, h, w, block, d), dtype=_BF16, device=x.device)
        pos = pos.to(_BF16).contiguous()
        if pos.shape != (h, block, d):
            raise RuntimeError("window positions must be 'h block d'")
        if w > 0:
            _lib.check(_lib.lib().nsa_windows_fwd(_ptr(x), _s3(x), _ptr(pos), b, h, n, d, int(block), int(stride), _ptr(out), _stream()), "nsa_windows_fwd")
        outs.append(out)
    return outs[0], outs[1]


@windows_pair_fwd.register_fake
def _(k, v, kpos, vpos, block, stride):
    b, h, n, d = k.shape
    return k.new_empty((b, h, n // stride, block, d)), v.new_empty((b, h, n // stride, block, d))


@torch.library.custom_op("nsa_amd::windows_pair_bwd", mutates_args=())
def windows_pair_bwd(dkw: Tensor, dvw: Tensor, n: int, stride: int) -> tuple[Tensor, Tensor]:
    outs = []
    for dwin in (dkw, dvw):
        dwin = dwin.contiguous()
        if dwin.dtype != _BF16:
            raise RuntimeError("window gradients must be bfloat16")
        b, h, w, block, d = dwin.shape
        dx = torch.empty((b, h, n, d), dtype=_BF16, device=dwin.device)
        if w == 0:
            dx.zero_()
        else:
            _lib.check(_lib.lib().nsa_windows_bwd(_ptr(dwin), b, h, n, d, block, int(stride), _ptr(dx), _stream()), "nsa_windows_bwd")
        outs.append(dx)
    return outs[0], outs[1]


@windows_pair_bwd.register_fake
def _(dkw, dvw, n, stride):
    b, h, w, block, d = dkw.shape
    return dkw.new_empty((b, h, n, d)), dvw.new_empty((b, h, n, d))


def _windows_pair_setup(ctx, inputs, output):
    k, v, kpos, vpos, block, stride = inputs
    ctx.n, ctx.stride = k.shape[2], stride
    ctx.pos_dtypes = (kpos.dtype, vpos.dtype)


def _windows_pair_backward(ctx, dkw, dvw):
    dkw = dkw if dkw.dtype == _BF16 else dkw.to(_BF16)
    dvw = dvw if dvw.dtype == _BF16 else dvw.to(_BF16)
    dk, dv = windows_pair_bwd(dkw, dvw, ctx.n, ctx.stride)
    dkpos = dkw.sum(dim=(0, 2), dtype=torch.float32).to(ctx.pos_dtypes[0])
    dvpos = dvw.sum(dim=(0, 2), dtype=torch.float32).to(ctx.pos_dtypes[1])
    return dk, dv, dkpos, dvpos, None, None


windows_pair_fwd.register_autograd(_windows_pair_backward, setup_context=_windows_pair_setup)


def compress_windows_pair(k: Tensor, v: Tensor, kpos: Tensor, vpos: Tensor, block: int, stride: int):
    """`compress_windows` of the keys and the values of a layer in one operator call."""
    d = k.shape[-1]
    D = _kernel_dim(d)
    kw, vw = windows_pair_fwd(_pad_dim(k, D), _pad_dim(v, D), _pad_dim(kpos, D), _pad_dim(vpos, D), int(block), int(stride))
    return kw[..., :d], vw[..., :d]


def compress_windows(x: Tensor, pos: Tensor | None, block: int, stride: int) -> Tensor:
    """'b h n d' -> 'b h w block d' with w = n // stride: window w = tokens (w+1)*stride - block ..
    (w+1)*stride - 1, zeros left of token 0, plus the intra-window positions 'h block d'
    (NSA.py:270-275, 589-603)."""
    d = x.shape[-1]
    D = _kernel_dim(d)
    out = windows_fwd(_pad_dim(x, D), None if pos is None else _pad_dim(pos, D), int(block), int(stride))
    return out[..., :d]


@torch.no_grad()
def decode_importance_topk(logits: Tensor, kv_heads: int, per_block: int, share: bool, num_selected: int):
    """Decode step: logits 'b hq nc' (from decode_range_attend) -> pooled over the `per_block`
    compressed keys of a selection block and, if `share`, over the heads of a kv group; padded
    softmax, top-k, mask (NSA.py:448-476, 502).  Returns (values, indices, mask) shaped
    'b hk 1 k' or 'b hq 1 k'."""
    if logits.dtype != torch.float32 or not logits.is_cuda or not logits.is_contiguous():
        raise RuntimeError("decode logits must be contiguous fp32 device tensors")
    b, hq, nc = logits.shape
    units = kv_heads if share else hq
    shp = (b, units, 1, int(num_selected))
    idx = torch.empty(shp, dtype=torch.int32, device=logits.device)
    vals = torch.empty(shp, dtype=torch.float32, device=logits.device)
    fm = torch.empty(shp, dtype=torch.uint8, device=logits.device)
    _lib.check(_lib.lib().nsa_decode_topk(_ptr(logits), b, int(kv_heads), hq // kv_heads, nc, int(per_block), int(bool(share)),
                                          int(num_selected), _ptr(idx), _ptr(vals), _ptr(fm), _stream()), "nsa_decode_topk")
    return vals, idx, fm.view(torch.bool)


@torch.no_grad()
def decode_step(q: Tensor, k: Tensor, v: Tensor, freqs: Tensor, pos: int, keys: Tensor, vals: Tensor, ck: Tensor | None, cv: Tensor | None,
                mem_k: Tensor | None, mem_v: Tensor | None, k_run_row: Tensor | None, v_run_row: Tensor | None, gate_logits: Tensor,
                *, per_block: int, block: int, num_sel: int, share: bool, window: int, scale: float | None = None):
    """The attention part of one decode step in a single library call (see nsa_decode_step in
    include/nsa_hip.h).  q 'b hq 1 d', k, v 'b hk 1 d': the new token's projections; keys, vals: the
    caches with row `pos` free ('b hk >=pos+1 d' views from the start of their buffers); ck, cv: the
    compressed caches (None or empty before the first compressed key); mem_k, mem_v 'hk m d'.
    Returns (merged 'b 1 (h d)', idx int32, fmask bool) with idx / fmask 'b hk|hq 1 k'."""
    q, k, v = _prep(q), _prep(k), _prep(v)
    b, hq, _, d = q.shape
    hk = k.shape[1]
    nc = 0 if ck is None else ck.shape[2]
    for t in (keys, vals) + ((ck, cv) if nc else ()):
        if t.dtype != _BF16 or not t.is_cuda or not _rows_ok(t):
            raise RuntimeError("decode_step: caches must be bf16 device tensors with unit feature stride and 16-byte aligned rows")
    if keys.shape[2] < pos + 1 or vals.shape[2] < pos + 1:
        raise RuntimeError("decode_step: the caches have no row for the new token")
    dsc = _lib.DecodeStepDesc()
    dsc.batch, dsc.heads, dsc.kv_heads, dsc.dim_head = b, hq, hk, d
    dsc.pos, dsc.num_compressed, dsc.per_block, dsc.block = int(pos), nc, int(per_block), int(block)
    dsc.num_sel, dsc.share, dsc.window, dsc.scale = int(num_sel), int(bool(share)), int(window), (d ** -0.5 if scale is None else float(scale))
    m = 0
    if nc and mem_k is not None:
        mem_k, mem_v = mem_k.to(_BF16).contiguous(), mem_v.to(_BF16).contiguous()
        m = mem_k.shape[-2]
    dsc.num_mem = m
    for name, t in (("q_stride", q), ("k_stride", k), ("v_stride", v)):
        getattr(dsc, name)[:] = (t.stride(0), t.stride(1))
    dsc.kc_stride[:] = keys.stride()[:3]
    dsc.vc_stride[:] = vals.stride()[:3]
    if nc:
        dsc.ck_stride[:] = ck.stride()[:3]
        dsc.cv_stride[:] = cv.stride()[:3]
    run = k_run_row is not None and v_run_row is not None
    if run:
        for t in (k_run_row, v_run_row):
            if t.dtype != _BF16 or t.shape != (b, hk, 1, d) or not _rows_ok(t):
                raise RuntimeError("decode_step: window rows must be bf16 'b hk 1 d' views")
        dsc.krun_stride[:] = (k_run_row.stride(0), k_run_row.stride(1))
        dsc.vrun_stride[:] = (v_run_row.stride(0), v_run_row.stride(1))
    L = _lib.lib()
    nbytes, ioff, foff, ksel = C.c_size_t(), C.c_size_t(), C.c_size_t(), C.c_int32()
    _lib.check(L.nsa_decode_step_workspace_bytes(C.byref(dsc), C.byref(nbytes), C.byref(ioff), C.byref(foff), C.byref(ksel)),
               "nsa_decode_step_workspace_bytes")
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=q.device)
    gl = gate_logits if gate_logits.dtype == _BF16 and gate_logits.is_contiguous() else gate_logits.to(_BF16).contiguous()
    if gl.numel() != b * hq * 3:
        raise RuntimeError("decode_step: gate logits must be 'b 1 (h 3)'")
    freqs = freqs.detach()
    if freqs.dtype != torch.float32 or not freqs.is_contiguous():
        freqs = freqs.to(torch.float32).contiguous()
    out = torch.empty((b, 1, hq * d), dtype=_BF16, device=q.device)
    _lib.check(L.nsa_decode_step(C.byref(dsc), _ptr(q), _ptr(k), _ptr(v), _ptr(freqs), _ptr(keys), _ptr(vals), _ptr(ck) if nc else None,
                                 _ptr(cv) if nc else None, _ptr(mem_k) if m else None, _ptr(mem_v) if m else None,
                                 _ptr(k_run_row) if run else None, _ptr(v_run_row) if run else None, _ptr(gl), _ptr(ws), nbytes, _ptr(out),
                                 _stream()), "nsa_decode_step")
    units = hk if share else hq
    kk = ksel.value
    idx = ws[ioff.value:ioff.value + b * units * kk * 4].view(torch.int32).view(b, units, 1, kk)
    fm = ws[foff.value:foff.value + b * units * kk].view(torch.bool).view(b, units, 1, kk)
    return out, idx, fm


# ------------------------------------------------------------- epilogue of the qkv projection

def qkv_prep_supported(qkv: Tensor, dim_head: int) -> bool:
    """The fused epilogue runs on device projections in bf16 or fp32 with 64 or 128 features per head, outside a compiler
    trace (it is a plain autograd.Function over the C ABI, not a registered operator)."""
    return (qkv.is_cuda and qkv.dtype in (_BF16, torch.float32) and dim_head in (64, 128) and qkv.dim() == 3
            and not torch.compiler.is_compiling())


def _qkv_desc(qkv: Tensor, heads: int, kv_heads: int, d: int, block: int, stride: int, offset: int) -> _lib.QkvDesc:
    dsc = _lib.QkvDesc()
    dsc.batch, dsc.seq, dsc.heads, dsc.kv_heads, dsc.dim_head = qkv.shape[0], qkv.shape[1], heads, kv_heads, d
    dsc.block, dsc.stride, dsc.fp32, dsc.offset = block, stride, int(qkv.dtype == torch.float32), offset
    dsc.qkv_stride[:] = (qkv.stride(0), qkv.stride(1))
    return dsc


class _QkvPrep(torch.autograd.Function):
    """One kernel over the qkv projection's output in each direction (see nsa_qkv_prep_fwd in include/nsa_hip.h)."""

    @staticmethod
    def forward(ctx, qkv, freqs, kpos, vpos, heads, kv_heads, d, block, stride, offset):
        b, n, width = qkv.shape
        if width != (heads + 2 * kv_heads) * d:
            raise RuntimeError(f"qkv projection of width {width}: expected (heads + 2 kv_heads) * dim_head = {(heads + 2 * kv_heads) * d}")
        if qkv.stride(2) != 1 or qkv.stride(1) % 8 or qkv.stride(0) % 8 or qkv.data_ptr() % 16:
            qkv = qkv.contiguous()
        fp32 = qkv.dtype == torch.float32
        dev = qkv.device
        freqs32 = freqs.detach().to(torch.float32).contiguous()
        w = n // stride if block > 0 else 0
        rq = torch.empty((b, heads, n, d), dtype=_BF16, device=dev)
        rk = torch.empty((b, kv_heads, n, d), dtype=_BF16, device=dev)
        kw = torch.empty((b, kv_heads, w, block, d), dtype=qkv.dtype, device=dev)
        vw = torch.empty_like(kw)
        if fp32:
            q16 = torch.empty((b, heads, n, d), dtype=_BF16, device=dev)
            v16 = torch.empty((b, kv_heads, n, d), dtype=_BF16, device=dev)
        else:
            # a bf16 projection is read in place: 'b n (h d) -> b h n d' views
            q16 = qkv[..., :heads * d].view(b, n, heads, d).permute(0, 2, 1, 3)
            v16 = qkv[..., (heads + kv_heads) * d:].view(b, n, kv_heads, d).permute(0, 2, 1, 3)
        kp = kpos.detach().to(qkv.dtype).contiguous() if w > 0 else None
        vp = vpos.detach().to(qkv.dtype).contiguous() if w > 0 else None
        dsc = _qkv_desc(qkv, heads, kv_heads, d, block, stride, offset)
        _lib.check(_lib.lib().nsa_qkv_prep_fwd(C.byref(dsc), _ptr(qkv), _ptr(freqs32), _ptr(kp), _ptr(vp), _ptr(q16) if fp32 else None,
                                               _ptr(rq), _ptr(rk), _ptr(v16) if fp32 else None, _ptr(kw) if w > 0 else None,
                                               _ptr(vw) if w > 0 else None, _stream()), "nsa_qkv_prep_fwd")
        ctx.save_for_backward(freqs32)
        ctx.meta = (tuple(qkv.shape), qkv.dtype, heads, kv_heads, d, block, stride, offset, kpos.dtype, vpos.dtype,
                    ctx.needs_input_grad[2], ctx.needs_input_grad[3])
        ctx.set_materialize_grads(False)
        return q16, rq, rk, v16, kw, vw

    @staticmethod
    def backward(ctx, dq16, drq, drk, dv16, dkw, dvw):
        (freqs32,) = ctx.saved_tensors
        shape, dtype, heads, kv_heads, d, block, stride, offset, kp_dtype, vp_dtype, kp_grad, vp_grad = ctx.meta
        b, n, _ = shape
        c16 = lambda t: None if t is None else (t if t.dtype == _BF16 else t.to(_BF16)).contiguous()
        cw = lambda t: None if t is None or t.numel() == 0 else (t if t.dtype == dtype else t.to(dtype)).contiguous()
        dq16, drq, drk, dv16, dkw, dvw = c16(dq16), c16(drq), c16(drk), c16(dv16), cw(dkw), cw(dvw)
        dqkv = torch.empty(shape, dtype=dtype, device=freqs32.device)
        dsc = _qkv_desc(dqkv, heads, kv_heads, d, block, stride, offset)
        _lib.check(_lib.lib().nsa_qkv_prep_bwd(C.byref(dsc), _ptr(dq16), _ptr(drq), _ptr(drk), _ptr(dv16), _ptr(dkw), _ptr(dvw),
                                               _ptr(freqs32), _ptr(dqkv), _stream()), "nsa_qkv_prep_bwd")
        pos_grad = lambda t, dt: window_position_grad(t, dt) if colsum_supported(t) else t.sum(dim=(0, 2), dtype=torch.float32).to(dt)
        dkp = pos_grad(dkw, kp_dtype) if kp_grad and dkw is not None else None
        dvp = pos_grad(dvw, vp_dtype) if vp_grad and dvw is not None else None
        return dqkv, None, dkp, dvp, None, None, None, None, None, None


def qkv_prep(qkv: Tensor, freqs: Tensor, k_positions: Tensor, v_positions: Tensor, heads: int, kv_heads: int, dim_head: int,
             compress_block_size: int, compress_stride: int, offset: int = 0):
    """Everything the attention branches read, from the fused projection 'b n ((heads + 2 kv_heads) d)' in one pass
    (NSA.py:583-614, 643): returns (q, rotated q, rotated k, v) as bf16 'b h n d' and the compression windows of k and v
    'b h w cbs d' (+ intra-window positions) in the projection's dtype.  For a bf16 projection q and v are views of it."""
    if not qkv_prep_supported(qkv, dim_head):
        raise RuntimeError("qkv_prep: needs a bf16 / fp32 device projection 'b n (h d)' with dim_head 64 or 128")
    return _QkvPrep.apply(qkv, freqs, k_positions, v_positions, int(heads), int(kv_heads), int(dim_head), int(compress_block_size),
                          int(compress_stride), int(offset))


# ------------------------------------------------------------------ norm and column sums

def capturing() -> bool:
    """A HIP graph is being recorded on the current stream."""
    return torch.cuda.is_available() and torch.cuda.is_current_stream_capturing()


def colsum_supported(x: Tensor) -> bool:
    """One pass + a reduce of per-work-group partials (two launches) pays from about half a million elements on; below that the
    library's one-launch sum is as fast and a step bound by its launches (a small model) is better off with one launch.
    While a graph is being recorded every size takes the kernel: the library's sum over many work-groups records a memset
    node, and on replays after the first its results were wrong here (bias gradients of 1e37 in a replayed training step)."""
    return bool(x.is_cuda and x.dtype == _BF16 and x.shape[-1] % 8 == 0 and x.numel() > 0 and (x.numel() >= (1 << 19) or capturing()))


def colsum(x: Tensor, out_dtype=None) -> Tensor:
    """Sum of a bf16 matrix '... c' over all leading axes in fp32, one pass over the matrix (the bias gradient of a projection)."""
    c = x.shape[-1]
    x2 = x.reshape(-1, c)
    if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    out = torch.empty((c,), dtype=out_dtype or x.dtype, device=x.device)
    L = _lib.lib()
    ws = torch.empty((max(L.nsa_colsum_workspace(x2.shape[0], c, 1), 4) // 4,), dtype=torch.float32, device=x.device)
    _lib.check(L.nsa_colsum(_ptr(x2), 1, 0, 1, 0, x2.shape[0], x2.stride(0), c, _ptr(out), int(out.dtype == torch.float32), _ptr(ws),
                            _stream()), "nsa_colsum")
    return out


def window_position_grad(dwin: Tensor, out_dtype) -> Tensor:
    """Gradient of the intra-window positions 'h j d' from the gradient of the windows 'b h w j d' (contiguous bf16): its sum
    over batch and windows (NSA.py:599-600 add the positions to every window)."""
    b, h, w, j, d = dwin.shape
    direct = out_dtype in (_BF16, torch.float32)            # the kernel rounds the fp32 sums to bf16 itself
    out = torch.empty((h, j, d), dtype=out_dtype if direct else torch.float32, device=dwin.device)
    L = _lib.lib()
    ws = torch.empty((max(L.nsa_colsum_workspace(b * w, j * d, h), 4) // 4,), dtype=torch.float32, device=dwin.device)
    _lib.check(L.nsa_colsum(_ptr(dwin), h, dwin.stride(1), b, dwin.stride(0), w, dwin.stride(2), j * d, _ptr(out),
                            int(out.dtype == torch.float32), _ptr(ws), _stream()), "nsa_colsum")
    return out if direct else out.to(out_dtype)


def rms_norm_supported(x: Tensor, weight: Tensor | None) -> bool:
    return bool(weight is not None and x.is_cuda and x.dtype == _BF16 and weight.dtype == _BF16 and x.shape[-1] % 8 == 0
                and x.shape[-1] <= 4096 and x.numel() > 0 and weight.shape == x.shape[-1:])


def _rms_rows(x: Tensor) -> Tensor:
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    return x2


def _rms_fwd(x2: Tensor, weight: Tensor, eps: float):
    rows, dim = x2.shape
    y = torch.empty((rows, dim), dtype=_BF16, device=x2.device)
    rstd = torch.empty((rows,), dtype=torch.float32, device=x2.device)
    _lib.check(_lib.lib().nsa_rmsnorm_fwd(rows, dim, _ptr(x2), x2.stride(0), _ptr(weight), eps, _ptr(y), _ptr(rstd), _stream()),
               "nsa_rmsnorm_fwd")
    return y, rstd


def _rms_bwd(x2: Tensor, weight: Tensor, rstd: Tensor, dy2: Tensor, want_dw: bool):
    rows, dim = x2.shape
    if not dy2.is_contiguous() or dy2.data_ptr() % 16:
        dy2 = dy2.clone(memory_format=torch.contiguous_format)
    dx = torch.empty((rows, dim), dtype=_BF16, device=x2.device)
    dw = part = None
    L = _lib.lib()
    if want_dw:
        dw = torch.empty((dim,), dtype=weight.dtype, device=x2.device)
        part = torch.empty((L.nsa_rmsnorm_partials(rows) * dim,), dtype=torch.float32, device=x2.device)
    _lib.check(L.nsa_rmsnorm_bwd(rows, dim, _ptr(x2), x2.stride(0), _ptr(weight), _ptr(rstd), _ptr(dy2), _ptr(dx), _ptr(dw), 0, _ptr(part),
                                 _stream()), "nsa_rmsnorm_bwd")
    return dx, dw


class _RmsNorm(torch.autograd.Function):
    """nn.RMSNorm over the last axis (NSA.py:230, 579) as one HBM-bound kernel in each direction (see nsa_rmsnorm_fwd)."""

    @staticmethod
    def forward(ctx, x, weight, eps):
        x2 = _rms_rows(x)
        w = weight.detach().contiguous()
        y, rstd = _rms_fwd(x2, w, eps)
        ctx.save_for_backward(x2, w, rstd)
        return y.view(x.shape)

    @staticmethod
    def backward(ctx, dy):
        x2, w, rstd = ctx.saved_tensors
        dx, dw = _rms_bwd(x2, w, rstd, dy.reshape(x2.shape), ctx.needs_input_grad[1])
        return dx.view(dy.shape), dw, None


def rms_norm(x: Tensor, weight: Tensor, eps: float | None = None) -> Tensor:
    """torch.nn.functional.rms_norm(x, (dim,), weight, eps) for a bf16 device tensor.  eps None, as nn.RMSNorm(dim) has it, is
    the machine epsilon of the type the norm is computed in - fp32 for a bf16 input, in the library's kernel as here."""
    if not rms_norm_supported(x, weight) or torch.compiler.is_compiling() or torch.is_autocast_enabled():
        return torch.nn.functional.rms_norm(x, x.shape[-1:], weight, eps)
    return _RmsNorm.apply(x, weight, float(torch.finfo(torch.float32).eps if eps is None else eps))


# ------------------------------------------------------------------ projections

def _wgrad_splits(rows: int, n_in: int, n_out: int, replayed: bool = False) -> int:
    """How many slices of the token axis the weight gradient 'o i' = dy^T x is cut into.  The library's GEMM gives one work-group
    per output tile the whole token axis: with a few dozen tiles of a small weight and tens of thousands of tokens most of the
    256 CUs idle (measured on 16384 tokens: 1024 x 1024 weight 109 us whole, 52 us in 8 slices + the sum; 48 x 1024 99 -> 31 us;
    on 8192 tokens every weight from 24 x 512 to 2048 x 512 takes 47-57 us whole - the time follows the token count, not the
    weight - and 30-35 us in 4 or 8 slices, launches included; a 2048 x 2048 weight over 4080 tokens has its 256 tiles already and
    is left whole, and at 4096 tokens the whole GEMM's 27-31 us are what the two launches of the sliced one cost).
    `replayed`: the launches are being recorded into a graph, where they cost nothing at replay; then 4096 tokens are cut as
    well (GPU time alone: 64 x 1024 weight 27 -> 10 us in 4 slices, 1024 x 1024 30 -> 23 us) and 16 slices are allowed."""
    if rows < (4096 if replayed else 8192):
        return 1
    tiles = -(-n_in // 128) * -(-n_out // 128)
    s = 16 if replayed else 8
    while s > 1 and (s * tiles > 768 or rows % s or rows // s < 1024):
        s //= 2
    return s if s >= 4 else 1


class _Linear(torch.autograd.Function):
    """F.linear whose weight gradient is a batched GEMM over slices of the token axis, summed in fp32 (see _wgrad_splits):
    the same products as the one GEMM autograd would launch (NSA.py:583 to_qkv, 853 to_strategy_combine, 858 combine_heads)."""

    @staticmethod
    def forward(ctx, x, w, b):
        ctx.save_for_backward(x, w)
        ctx.has_bias = b is not None
        return torch.nn.functional.linear(x, w, b)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        n_out, n_in = w.shape
        dy2, x2 = dy.reshape(-1, n_out), x.reshape(-1, n_in)
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = (dy2 @ w).view(x.shape)
        if ctx.needs_input_grad[1]:
            dw = _wgrad(dy2, x2, w.dtype)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = colsum(dy2) if colsum_supported(dy2) else dy2.sum(0)
        return dx, dw, db


def linear(x: Tensor, weight: Tensor, bias: Tensor | None = None) -> Tensor:
    """torch.nn.functional.linear with the split weight-gradient GEMM (see _Linear)."""
    if (not (torch.is_grad_enabled() and weight.requires_grad) or torch.compiler.is_compiling() or x.dtype != weight.dtype
            or torch.is_autocast_enabled()):               # under autocast the library casts the operands itself
        return torch.nn.functional.linear(x, weight, bias)
    return _Linear.apply(x, weight, bias)


def _wgrad(dy2: Tensor, x2: Tensor, dtype) -> Tensor:
    """Weight gradient 'o i' = dy2^T x2 of a projection, over slices of the token axis where that fills the chip."""
    rows, n_in, n_out = x2.shape[0], x2.shape[1], dy2.shape[1]
    s = _wgrad_splits(rows, n_in, n_out, capturing()) if x2.is_cuda and x2.dtype in (_BF16, torch.float16) and dy2.dtype == x2.dtype else 1
    if s > 1 and dy2.is_contiguous() and x2.is_contiguous():
        try:
            part = torch.bmm(dy2.view(s, rows // s, n_out).transpose(1, 2), x2.view(s, rows // s, n_in), out_dtype=torch.float32)
        except TypeError:                     # a torch without fp32 output from a bf16 batched GEMM: partial products in bf16
            part = torch.bmm(dy2.view(s, rows // s, n_out).transpose(1, 2), x2.view(s, rows // s, n_in)).float()
        if dtype not in (_BF16, torch.float32) or (n_out * n_in) % 4:
            return part.sum(0).to(dtype)
        dw = torch.empty((n_out, n_in), dtype=dtype, device=x2.device)
        _lib.check(_lib.lib().nsa_sum_slices(_ptr(part), s, n_out * n_in, _ptr(dw), int(dtype == torch.float32), _stream()), "nsa_sum_slices")
        return dw
    return (dy2.t() @ x2).to(dtype)


class _NormedProjections(torch.autograd.Function):
    """The module's front end as one node: RMS norm of the input (NSA.py:579), the fused q / k / v projection (NSA.py:583) and the
    gate logits (NSA.py:853) of the normed input.  One node so that the two gradients of the normed input are accumulated by the
    second GEMM (beta = 1) instead of an extra pass over them, and the norm's backward is one kernel."""

    @staticmethod
    def forward(ctx, inp, norm_w, eps, w_qkv, w_gate, b_gate):
        x2 = _rms_rows(inp)
        nw = norm_w.detach().contiguous()
        xn, rstd = _rms_fwd(x2, nw, eps)
        qkv = xn @ w_qkv.t()
        logits = torch.addmm(b_gate, xn, w_gate.t()) if b_gate is not None else xn @ w_gate.t()
        ctx.save_for_backward(x2, nw, rstd, xn, w_qkv, w_gate)
        ctx.has_bias = b_gate is not None
        lead = inp.shape[:-1]
        return qkv.view(*lead, -1), logits.view(*lead, -1)

    @staticmethod
    def backward(ctx, dqkv, dlogits):
        x2, nw, rstd, xn, w_qkv, w_gate = ctx.saved_tensors
        dq2 = dqkv.reshape(-1, w_qkv.shape[0])
        dl2 = dlogits.reshape(-1, w_gate.shape[0])
        need = ctx.needs_input_grad
        dinp = dnw = dwq = dwg = dbg = None
        if need[0] or need[1]:
            dxn = dq2 @ w_qkv
            dxn.addmm_(dl2, w_gate)
            dinp, dnw = _rms_bwd(x2, nw, rstd, dxn, need[1])
            dinp = dinp.view(*dqkv.shape[:-1], -1) if need[0] else None
        if need[3]:
            dwq = _wgrad(dq2 if dq2.is_contiguous() else dq2.contiguous(), xn, w_qkv.dtype)
        if need[4]:
            dwg = _wgrad(dl2 if dl2.is_contiguous() else dl2.contiguous(), xn, w_gate.dtype)
        if ctx.has_bias and need[5]:
            dbg = colsum(dl2) if colsum_supported(dl2) else dl2.sum(0)
        return dinp, dnw, None, dwq, dwg, dbg


def normed_projections(inp: Tensor, norm_weight: Tensor, eps: float | None, w_qkv: Tensor, w_gate: Tensor, b_gate: Tensor | None):
    """(to_qkv(norm(inp)), gate_logits(norm(inp))) for a bf16 module with gradients (see _NormedProjections)."""
    return _NormedProjections.apply(inp, norm_weight, float(torch.finfo(torch.float32).eps if eps is None else eps), w_qkv, w_gate, b_gate)


# ------------------------------------------------------------------ fp32 forward

class _Fp32ValueBf16Grad(torch.autograd.Function):
    """An attention branch of an fp32 module under autograd.  The fp32 kernels are forward kernels; there is no fp32 backward.
    The forward value is theirs (the reference's fp32 bound, 1e-5, holds with gradients enabled too, so the parallel forward
    and the decode steps of tests/test_sparse_attn.py:50-91 agree whatever the grad mode); the gradient is the gradient of
    the same branch evaluated by the bf16 kernels on the bf16-rounded inputs (forward + backward, run in `backward`), which
    meets the gradient bound of a bf16 run (5e-2).  `fwd32(*tensors)` and `fwd16(*tensors)` evaluate the branch; every tensor
    argument is a candidate for a gradient."""

    @staticmethod
    def forward(ctx, fwd32, fwd16, *tensors):
        ctx.fwd16 = fwd16
        ctx.save_for_backward(*tensors)
        return fwd32(*tensors)

    @staticmethod
    def backward(ctx, dout):
        tensors = ctx.saved_tensors
        need = ctx.needs_input_grad[2:]
        with torch.enable_grad():
            ins = [t.detach().to(_BF16).requires_grad_(bool(nd)) for t, nd in zip(tensors, need)]
            out = ctx.fwd16(*ins)
            wanted = [t for t in ins if t.requires_grad]
            grads = iter(torch.autograd.grad(out, wanted, dout.to(out.dtype), allow_unused=True)) if wanted else iter(())
        res = []
        for t, nd in zip(tensors, need):
            g = next(grads) if nd else None
            res.append(None if g is None else g.to(t.dtype))
        return (None, None, *res)


def fp32_value_bf16_grad(fwd32, fwd16, *tensors: Tensor) -> Tensor:
    """`fwd32(*tensors)` (fp32 kernels), differentiable through `fwd16` (bf16 kernels) when gradients are being recorded."""
    if torch.is_grad_enabled() and any(t.requires_grad for t in tensors):
        return _Fp32ValueBf16Grad.apply(fwd32, fwd16, *tensors)
    with torch.no_grad():
        return fwd32(*tensors)


def _f32(t: Tensor) -> Tensor:
    if t.dtype != torch.float32 or not t.is_cuda:
        raise RuntimeError("the fp32 forward kernels take fp32 device tensors")
    ok = t.stride(-1) == 1 and all(st % 4 == 0 for st in t.stride()[:-1]) and t.data_ptr() % 16 == 0
    return t if ok else t.contiguous()


def _check_f32_dim(d: int):
    if d > 128 or d % 4:
        raise RuntimeError(f"dim_head {d}: the fp32 forward kernels take head dimensions <= 128 that are multiples of 4")


@torch.no_grad()
def dense_attend_f32(q: Tensor, k: Tensor, v: Tensor, mode: int, causal: bool, window: int = 0, stride: int = 1, num_mem: int = 0,
                     q_offset: int = 0):
    """Sliding-window (mode 0) or compressed (mode 1: k / v = [memory rows; compressed keys]) attention evaluated in fp32
    (NSA.py:841-850 / 621-639).  q 'b hq n d', k / v 'b hk rows d', any group size; query row i sits at position
    i + q_offset (a decode step: one row at the cached length).  Returns (out 'b hq n d', lse)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    b, hq, n, d = q.shape
    _check_f32_dim(d)
    out = torch.empty((b, hq, n, d), dtype=torch.float32, device=q.device)
    lse = torch.empty((b, hq, n), dtype=torch.float32, device=q.device)
    dsc = _dense_desc(q, k, v, out, out, int(mode), bool(causal), int(window), int(stride), int(num_mem), False, 1, True, float(d ** -0.5))
    _lib.check(_lib.lib().nsa_dense_fwd_f32(C.byref(dsc), _ptr(q), _ptr(k), _ptr(v), _ptr(out), _ptr(lse), int(q_offset), _stream()),
               "nsa_dense_fwd_f32")
    return out, lse


@torch.no_grad()
def native_sparse_attend_f32(fq: Tensor, fk: Tensor, fv: Tensor, block_size: int, selected_block_indices: Tensor, fmask: Tensor,
                             include_block_causal: bool = True, return_lse: bool = False, q_offset: int = 0):
    """`native_sparse_attend` evaluated in fp32 (forward only): same arguments and contract (TRI.py:1938-1987, NSA.py:741-819),
    any block size, any group size.  fq may hold fewer rows than fk / fv: row i is the query at position i + q_offset."""
    q_heads, kv_heads, sel_heads = fq.shape[1], fk.shape[1], selected_block_indices.shape[1]
    assert q_heads % kv_heads == 0 and sel_heads in (q_heads, kv_heads)
    d = fq.shape[-1]
    _check_f32_dim(d)
    if kv_heads != sel_heads:
        fk, fv = fk.repeat_interleave(q_heads // kv_heads, dim=1), fv.repeat_interleave(q_heads // kv_heads, dim=1)
    q, k, v = _f32(fq), _f32(fk), _f32(fv)
    b, hq, n, _ = q.shape
    idx = selected_block_indices.contiguous()
    if idx.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("selected_block_indices must be int64 or int32")
    fm = fmask.contiguous().view(torch.uint8) if fmask.dtype == torch.bool else fmask.contiguous().to(torch.uint8)
    out = torch.empty((b, hq, n, d), dtype=torch.float32, device=q.device)
    lse = torch.empty((b, hq, n), dtype=torch.float32, device=q.device)
    dsc = _select_desc(q, k, v, out, idx.shape[-1], int(block_size), bool(include_block_causal), float(d ** -0.5), idx.dtype == torch.int64)
    _lib.check(_lib.lib().nsa_select_fwd_f32(C.byref(dsc), _ptr(q), _ptr(k), _ptr(v), _ptr(idx) if idx.numel() else None,
                                             _ptr(fm) if fm.numel() else None, _ptr(out), _ptr(lse), k.shape[2], int(q_offset), _stream()),
               "nsa_select_fwd_f32")
    if not include_block_causal and idx.shape[-1] > 0 and q_offset == 0 and k.shape[2] == n:
        out = _dead_rows_uniform(out, fv, selected_block_indices, fmask, int(block_size), q_heads, d)
    return (out, lse) if return_lse else out


def importance_logits_f32(q: Tensor, ck: Tensor, stride: int, sel_block: int, share: bool, causal: bool, mask_own: bool = True):
    """Block-importance logits of NSA.py:652-691 in fp32.  They are the mean, over a fine block's compressed keys and (if
    shared) the group's heads, of scale * q . ck - linear in both, so one fp32 GEMM against the block means of the
    compressed keys `ck` 'b hk nc d' (memory slots excluded); -inf where the reference's fill values remove the block from
    the softmax (a block not entirely before the query; the query's own block when stride != sel_block).  None when no
    full fine block exists.  Plain torch, differentiable in q and ck."""
    b, hq, n, d = q.shape
    hk = ck.shape[1]
    g = hq // hk
    npf = sel_block // stride
    nb = ck.shape[2] // npf
    if nb == 0:
        return None
    cbar = ck[:, :, :nb * npf].float().reshape(b, hk, nb, npf, d).mean(dim=3)
    qq = q.float().reshape(b, hk, g, n, d).mean(dim=2) if share else q.float()
    if not share:
        cbar = cbar.repeat_interleave(g, dim=1)
    imp = torch.matmul(qq, cbar.transpose(-1, -2)) * (d ** -0.5)
    i = torch.arange(n, device=q.device)[:, None]
    j = torch.arange(nb, device=q.device)[None, :]
    dead = torch.zeros((n, nb), dtype=torch.bool, device=q.device)
    if causal:
        dead |= (j + 1) * sel_block > i
    if stride != sel_block and mask_own:      # decode steps (mask_own False): every cached block lies before the query
        dead |= (i // sel_block) == j
    return imp.masked_fill(dead, float("-inf"))


@torch.no_grad()
def qkv_prep_f32(qkv: Tensor, freqs: Tensor, k_positions: Tensor, v_positions: Tensor, heads: int, kv_heads: int, dim_head: int,
                 compress_block_size: int, compress_stride: int, offset: int = 0):
    """`qkv_prep` for the fp32 forward: (q, rotated q, rotated k, v, k windows, v windows), all fp32; q and v are views of
    the projection.  dim_head 64 or 128."""
    if qkv.dtype != torch.float32 or dim_head not in (64, 128) or not qkv.is_cuda:
        raise RuntimeError("qkv_prep_f32: needs an fp32 device projection with dim_head 64 or 128")
    b, n, width = qkv.shape
    heads, kv_heads, d, block, stride = int(heads), int(kv_heads), int(dim_head), int(compress_block_size), int(compress_stride)
    if qkv.stride(2) != 1 or qkv.stride(1) % 8 or qkv.stride(0) % 8 or qkv.data_ptr() % 16:
        qkv = qkv.contiguous()
    w = n // stride if block > 0 else 0
    rq = torch.empty((b, heads, n, d), dtype=torch.float32, device=qkv.device)
    rk = torch.empty((b, kv_heads, n, d), dtype=torch.float32, device=qkv.device)
    kw = torch.empty((b, kv_heads, w, block, d), dtype=torch.float32, device=qkv.device)
    vw = torch.empty_like(kw)
    freqs32 = freqs.detach().to(torch.float32).contiguous()
    kp = k_positions.detach().to(torch.float32).contiguous() if w > 0 else None
    vp = v_positions.detach().to(torch.float32).contiguous() if w > 0 else None
    dsc = _qkv_desc(qkv, heads, kv_heads, d, block, stride, int(offset))
    dsc.fp32 = 2
    _lib.check(_lib.lib().nsa_qkv_prep_fwd(C.byref(dsc), _ptr(qkv), _ptr(freqs32), _ptr(kp), _ptr(vp), None, _ptr(rq), _ptr(rk), None,
                                           _ptr(kw) if w > 0 else None, _ptr(vw) if w > 0 else None, _stream()), "nsa_qkv_prep_fwd")
    q = qkv[..., :heads * d].view(b, n, heads, d).permute(0, 2, 1, 3)
    v = qkv[..., (heads + kv_heads) * d:].view(b, n, kv_heads, d).permute(0, 2, 1, 3)
    return q, rq, rk, v, kw, vw
