"""Parity of the sliding-window, compressed (+ importance logits), top-k and gate kernels
(through the C ABI) against the CPU oracle.  Forward 2e-2 abs / 1e-2 rel, gradients 5e-2 rel
(BASELINE.json); top-k indices bit-exact on identical scores."""
import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import assert_close, assert_grad_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rand(shape, g, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def _grad_close(got, want, name):
    assert_grad_close(got, want, name)


SLIDING = [
    # b, hq, hk, n, d, win, causal
    (2, 4, 2, 300, 64, 32, True),
    (1, 8, 2, 700, 128, 100, True),
    (1, 4, 4, 257, 64, 512, True),        # window >= n: full causal attention
    (2, 4, 1, 200, 64, 17, False),
    (1, 16, 4, 1024, 64, 64, True),
    (1, 6, 2, 200, 64, 32, True),         # G=3: not a power of two (padded with zero heads)
    (1, 4, 2, 150, 32, 20, True),         # dim_head 32 (zero-padded to 64)
    (1, 2, 1, 150, 96, 20, False),        # dim_head 96 (-> 128)
    (1, 4, 2, 500, 128, 70, False),       # d 128, window on both sides, several key tiles, the last one partial
]


@pytest.mark.parametrize("b,hq,hk,n,d,win,causal", SLIDING)
def test_sliding_matches_oracle(b, hq, hk, n, d, win, causal):
    from native_sparse_attention_pytorch_amd.ops import sliding_attend
    print(f"sliding b={b} hq={hq} hk={hk} n={n} d={d} win={win} causal={causal}", flush=True)
    g = torch.Generator().manual_seed(n + win)
    q, k, v, do = _rand((b, hq, n, d), g, d ** -0.25), _rand((b, hk, n, d), g, d ** -0.25), _rand((b, hk, n, d), g), _rand((b, hq, n, d), g)
    qr, kr, vr = (t.float().requires_grad_() for t in (q, k, v))
    ref = O.sliding_attend(qr, kr, vr, win, causal=causal)
    (ref * do.float()).sum().backward()
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    out = sliding_attend(qg, kg, vg, win, causal=causal)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert_close(out, ref, 2e-2, 1e-2, "sliding out")
    _grad_close(qg.grad, qr.grad, "dq")
    _grad_close(kg.grad, kr.grad, "dk")
    _grad_close(vg.grad, vr.grad, "dv")


@pytest.mark.parametrize("mode", ["sliding", "compressed"])
def test_dkv_ignores_rows_past_the_sequence_end(mode):
    """d = 128 dK/dV walk, n not a multiple of the 8-query tile of a group of 4, contiguous q / dO: the padding rows of a
    ragged last tile of head g alias the leading rows of head g + 1.  They must add nothing to dK / dV whatever (finite)
    values sit there: large values in the first rows of every head but the first leave the gradients at the oracle's."""
    from native_sparse_attention_pytorch_amd.ops import sliding_attend, compress_attend
    b, hq, hk, n, d = 1, 8, 2, 203, 128
    g = torch.Generator().manual_seed(7)
    q, do = _rand((b, hq, n, d), g, d ** -0.25), _rand((b, hq, n, d), g)
    with torch.no_grad():
        q[:, 1:, :8] *= 64.0            # (finite, far larger than anything else; scores of those rows saturate the softmax)
        do[:, 1:, :8] *= 512.0
    if mode == "sliding":
        k, v = _rand((b, hk, n, d), g, d ** -0.25), _rand((b, hk, n, d), g)
    else:
        k, v = _rand((b, hk, 1 + n // 4, d), g, d ** -0.25), _rand((b, hk, 1 + n // 4, d), g)
    qr, kr, vr = (t.float().requires_grad_() for t in (q, k, v))
    if mode == "sliding":
        ref = O.sliding_attend(qr, kr, vr, 40, causal=True)
    else:
        ref = O.attend(qr, kr, vr, mask=O.compress_mask(n, n // 4, 4, 1, True))
    (ref * do.float()).sum().backward()
    qg, kg, vg = (t.to(DEV).contiguous().requires_grad_() for t in (q, k, v))
    out = sliding_attend(qg, kg, vg, 40, causal=True) if mode == "sliding" else compress_attend(qg, kg, vg, 1, 4, True)[0]
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert torch.isfinite(kg.grad.float()).all() and torch.isfinite(vg.grad.float()).all()
    _grad_close(kg.grad, kr.grad, "dk")
    _grad_close(vg.grad, vr.grad, "dv")


COMPRESS = [
    # b, hq, hk, n, d, st, B, mem, causal, share
    (2, 4, 2, 200, 64, 4, 16, 1, True, True),
    (1, 8, 2, 515, 128, 16, 64, 1, True, True),      # config-3/4 geometry: st 16, B 64 -> npf 4
    (1, 4, 4, 130, 64, 8, 8, 2, True, True),         # stride == block (npf 1), two memory slots
    (1, 4, 2, 96, 64, 2, 16, 1, False, True),        # non-causal, npf 8
    (1, 4, 2, 160, 64, 4, 32, 1, True, False),       # per-head selection (no group mean)
    (1, 8, 2, 40, 64, 16, 64, 1, True, True),        # n < B: no full fine block
    (1, 4, 2, 3, 64, 4, 16, 1, True, True),          # n < stride: only the memory slot
    (1, 4, 2, 300, 64, 2, 32, 1, True, True),        # npf 16
    (1, 4, 2, 333, 64, 4, 20, 1, True, True),        # npf 5 (selection block 20: the reference's inference test grid)
    (1, 4, 2, 150, 64, 2, 20, 2, True, False),       # npf 10, per-head selection
    (1, 4, 2, 100, 64, 4, 12, 1, False, True),       # npf 3, non-causal
    (1, 6, 2, 200, 64, 4, 16, 1, True, True),        # G=3, shared selection: the group mean must be over 3 heads
    (1, 6, 2, 200, 64, 4, 16, 1, True, False),       # G=3, per-head selection
    (1, 12, 2, 100, 64, 4, 20, 1, True, True),       # G=6 with npf 5
    (1, 4, 2, 200, 32, 4, 16, 1, True, True),        # dim_head 32
    (1, 4, 2, 200, 96, 8, 16, 2, True, False),       # dim_head 96
    (1, 8, 2, 2100, 128, 8, 32, 2, True, True),      # d 128, 262 compressed keys + 2 slots: full tiles, a partial last tile, npf 4
    (1, 4, 2, 1100, 128, 4, 16, 1, False, True),     # d 128, non-causal: every query tile walks all 5 key tiles
]


@pytest.mark.parametrize("b,hq,hk,n,d,st,B,mem,causal,share", COMPRESS)
def test_compress_matches_oracle(b, hq, hk, n, d, st, B, mem, causal, share):
    from native_sparse_attention_pytorch_amd.ops import compress_attend
    print(f"compress b={b} hq={hq} hk={hk} n={n} d={d} st={st} B={B} mem={mem} causal={causal} share={share}", flush=True)
    g = torch.Generator().manual_seed(n * 7 + st)
    nc = n // st
    q = _rand((b, hq, n, d), g, d ** -0.25)
    ck, cv = _rand((b, hk, mem + nc, d), g, d ** -0.25), _rand((b, hk, mem + nc, d), g)
    do = _rand((b, hq, n, d), g)
    qr, kr, vr = (t.float().requires_grad_() for t in (q, ck, cv))
    cm = O.compress_mask(n, nc, st, mem, causal) if causal else None
    ref, csim = O.attend(qr, kr, vr, mask=cm, return_sim=True)
    (ref * do.float()).sum().backward()
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, ck, cv))
    out, imp = compress_attend(qg, kg, vg, mem, st, causal, sel_block=B, share=share)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert_close(out, ref, 2e-2, 1e-2, "compressed out")
    _grad_close(qg.grad, qr.grad, "dq")
    _grad_close(kg.grad, kr.grad, "dck (incl. memory slots)")
    _grad_close(vg.grad, vr.grad, "dcv")
    want = O.importance_logits(csim.detach(), mem, hq // hk, share, st, B)
    if want.shape[-1] == 0:
        assert imp is None
        return
    imp = imp.cpu()
    assert imp.shape == want.shape
    dead = want < -1e30
    assert torch.equal(torch.isinf(imp) & (imp < 0), dead), "set of unselectable blocks differs"
    assert_close(imp[~dead], want[~dead], 2e-3, 1e-3, "importance logits")


def test_importance_logits_gradient_matches_oracle():
    """gradient of the importance logits with respect to q and the compressed keys (needed by the
    differentiable top-k, NSA.py:715) against autograd through the oracle's NSA.py:652-691."""
    from native_sparse_attention_pytorch_amd.ops import compress_attend
    for (b, hq, hk, n, d, st, B, mem, share) in [(1, 4, 2, 200, 64, 4, 16, 1, True), (1, 4, 2, 160, 64, 4, 32, 2, False)]:
        g = torch.Generator().manual_seed(n)
        nc = n // st
        q = _rand((b, hq, n, d), g, d ** -0.25)
        ck, cv = _rand((b, hk, mem + nc, d), g, d ** -0.25), _rand((b, hk, mem + nc, d), g)
        qr, kr = q.float().requires_grad_(), ck.float().requires_grad_()
        _, csim = O.attend(qr, kr, cv.float(), mask=O.compress_mask(n, nc, st, mem, True), return_sim=True)
        want = O.importance_logits(csim, mem, hq // hk, share, st, B)
        w = torch.randn(want.shape, generator=g)
        live = want > -1e30
        (want * w).masked_fill(~live, 0.0).sum().backward()
        qg, kg = q.to(DEV).requires_grad_(), ck.to(DEV).requires_grad_()
        _, imp = compress_attend(qg, kg, cv.to(DEV), mem, st, True, sel_block=B, share=share)
        (imp * w.to(DEV)).masked_fill(~live.to(DEV), 0.0).sum().backward()
        torch.cuda.synchronize()
        _grad_close(qg.grad, qr.grad, "dq via importance")
        _grad_close(kg.grad, kr.grad, "dck via importance")


def test_topk_bit_exact_on_given_scores():
    from native_sparse_attention_pytorch_amd.ops import topk_op
    g = torch.Generator().manual_seed(0)
    for nb, k in [(5, 2), (64, 16), (100, 16), (512, 16), (700, 9), (33, 33), (128, 16), (256, 7), (300, 12), (510, 16), (64, 1), (17, 16)]:
        s = torch.rand(3, 2, 50, nb, generator=g)
        s = (s * 8).round() / 8 if nb % 2 == 0 else s           # many exact ties on even sizes
        s[0, 0, :5] = 0.0                                        # all-zero rows (early queries)
        idx, vals, fm = topk_op(s.to(DEV), k, False)
        wv, wi = O.topk_lower_index_first(s, k)
        assert torch.equal(idx.cpu().long(), wi), f"indices differ nb={nb} k={k}"
        assert torch.equal(vals.cpu(), wv)
        assert torch.equal(fm.cpu().bool(), wv > 1e-10)


def test_topk_prefix_equals_topk_on_filled_logits():
    """nsa_topk_prefix on logits whose undefined part holds garbage (NaN) = nsa_topk on the same logits with -inf there,
    bit for bit (indices, values, mask): both kernel families (<= 512 blocks with k <= 16, and the general one), rows that
    see nothing, rows whose limit is not a multiple of 4, limits beyond the number of blocks."""
    from native_sparse_attention_pytorch_amd.ops import importance_topk
    g = torch.Generator().manual_seed(2)
    for b, h, n, nb, k, B in [(2, 2, 600, 37, 8, 16), (1, 3, 1000, 512, 16, 2), (1, 2, 700, 600, 16, 1), (2, 1, 300, 64, 20, 4), (1, 1, 130, 8, 8, 16)]:
        logits = torch.randn(b, h, n, nb, generator=g) * 2
        lim = (torch.arange(n) // B)[:, None]
        dead = torch.arange(nb)[None, :] >= lim
        full = logits.masked_fill(dead, float('-inf')).to(DEV)
        junk = logits.masked_fill(dead, float('nan')).to(DEV)
        v1, i1, f1 = importance_topk(full, k)
        v2, i2, f2 = importance_topk(junk, k, prefix=(n, B))
        assert torch.equal(i1, i2) and torch.equal(f1, f2), f"nb={nb} k={k} B={B}"
        assert torch.equal(v1, v2)


@pytest.mark.parametrize("hq,hk,n,d,st,B,mem,share", [(8, 2, 515, 128, 16, 64, 1, True), (4, 2, 700, 64, 4, 16, 2, True), (4, 2, 300, 64, 8, 8, 1, False)])
def test_compress_prefix_logits_select_the_same_blocks(hq, hk, n, d, st, B, mem, share):
    """The module's path without differentiable top-k (logits written and read below each row's causal limit only) against
    the full logits: same output, same selected blocks and mask."""
    from native_sparse_attention_pytorch_amd.ops import compress_attend, importance_topk
    g = torch.Generator().manual_seed(n + st)
    nc = n // st
    q = _rand((1, hq, n, d), g, d ** -0.25).to(DEV)
    ck, cv = _rand((1, hk, nc + mem, d), g, d ** -0.25).to(DEV), _rand((1, hk, nc + mem, d), g).to(DEV)
    o1, imp1 = compress_attend(q, ck, cv, mem, st, True, sel_block=B, share=share)
    o2, imp2, prefix = compress_attend(q, ck, cv, mem, st, True, sel_block=B, share=share, prefix_only=True)
    assert prefix == (n, B)
    assert torch.equal(o1, o2)
    k = min(6, imp1.shape[-1])
    v1, i1, f1 = importance_topk(imp1, k)
    v2, i2, f2 = importance_topk(imp2, k, prefix=prefix)
    assert torch.equal(i1, i2) and torch.equal(f1, f2) and torch.equal(v1, v2)


def test_importance_softmax_topk_matches_oracle():
    from native_sparse_attention_pytorch_amd.ops import importance_topk
    g = torch.Generator().manual_seed(1)
    b, h, n, nb, k, B = 2, 2, 600, 37, 8, 16
    logits = torch.randn(b, h, n, nb, generator=g) * 2
    blk = (torch.arange(n) // B)[:, None]
    logits = logits.masked_fill(torch.arange(nb)[None, :] >= blk, float('-inf'))       # causal visibility
    vals, idx, fm = importance_topk(logits.to(DEV), k)
    ref_p = O.importance_softmax(logits.masked_fill(torch.isinf(logits), -3.4e37))
    wv, wi = O.topk_lower_index_first(ref_p, k)
    assert_close(vals, wv, 1e-6, 1e-4, "top-k values")
    live = wv > 1e-10
    assert torch.equal(fm.cpu(), live)
    # indices must agree wherever the oracle's ordering is not a near-tie
    gap_ok = torch.ones_like(live)
    gap_ok[..., :-1] &= (wv[..., :-1] - wv[..., 1:]) > 1e-6 * wv[..., :-1].clamp_min(1e-30)
    gap_ok[..., 1:] &= (wv[..., :-1] - wv[..., 1:]) > 1e-6 * wv[..., :-1].clamp_min(1e-30)
    sel = live & gap_ok
    assert torch.equal(idx.cpu().long()[sel], wi[sel])
    assert sel.float().mean() > 0.5
    # rows with nothing visible: every slot dead
    assert not fm.cpu()[:, :, :B].any()


@pytest.mark.parametrize("d", [64, 128])
def test_dense_strided_views_equal_contiguous(d):
    """q / k / v as 'b n (h d) -> b h n d' views of one projection output (token stride = the whole row, k and v at
    offsets that are only 16-byte aligned): the tile copies address rows through the strides they are given, so the
    results must be bit-equal to those on contiguous copies, forward and backward, causal and two-sided windows."""
    from native_sparse_attention_pytorch_amd import ops
    b, hq, hk, n = 2, 8, 2, 777
    g = torch.Generator().manual_seed(d)
    big = _rand((b, n, (hq + 2 * hk) * d + 24), g, d ** -0.5).cuda()
    q = big[..., :hq * d].view(b, n, hq, d).transpose(1, 2)
    k = big[..., hq * d + 8:hq * d + 8 + hk * d].view(b, n, hk, d).transpose(1, 2)
    v = big[..., hq * d + 16 + hk * d:hq * d + 16 + 2 * hk * d].view(b, n, hk, d).transpose(1, 2)
    do = _rand((b, hq, n, d), g).cuda()
    for causal, win in ((True, 100), (False, 50)):
        o1, l1, _ = ops.dense_fwd(q, k, v, 0, causal, win, 1, 0, False, 1, True, d ** -0.5)
        o2, l2, _ = ops.dense_fwd(q.contiguous(), k.contiguous(), v.contiguous(), 0, causal, win, 1, 0, False, 1, True, d ** -0.5)
        assert torch.equal(o1, o2) and torch.equal(l1, l2)
        g1 = ops.dense_bwd(q, k, v, o1, do, l1, 0, causal, win, 1, 0, d ** -0.5)
        g2 = ops.dense_bwd(q.contiguous(), k.contiguous(), v.contiguous(), o2, do, l2, 0, causal, win, 1, 0, d ** -0.5)
        for a, b_ in zip(g1, g2):
            assert torch.equal(a, b_)


def test_dense_backward_with_query_heads_2gb_apart():
    """The d = 128 dK / dV kernel stages its Q / dO rows through buffer loads whose 32-bit offsets span the query heads of one
    kv head; heads further apart than that take the kernel with 64-bit addresses.  Same gradients either way."""
    from native_sparse_attention_pytorch_amd import ops
    hq, hk, n, d = 2, 1, 200, 128
    g = torch.Generator().manual_seed(9)
    far = (1 << 30) + 64
    big = torch.empty(far + n * d, dtype=torch.bfloat16, device=DEV)
    q = big.as_strided((1, hq, n, d), (0, far, d, 1))
    qc = _rand((1, hq, n, d), g, d ** -0.5).cuda()
    q.copy_(qc)
    k, v = _rand((1, hk, n, d), g, d ** -0.5).cuda(), _rand((1, hk, n, d), g).cuda()
    do = _rand((1, hq, n, d), g).cuda()
    o1, l1, _ = ops.dense_fwd(q, k, v, 0, True, 64, 1, 0, False, 1, True, d ** -0.5)
    o2, l2, _ = ops.dense_fwd(qc, k, v, 0, True, 64, 1, 0, False, 1, True, d ** -0.5)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    g1 = ops.dense_bwd(q, k, v, o1, do, l1, 0, True, 64, 1, 0, d ** -0.5)
    g2 = ops.dense_bwd(qc, k, v, o2, do, l2, 0, True, 64, 1, 0, d ** -0.5)
    for name, a, b_ in zip(("dq", "dk", "dv"), g1, g2):
        assert_close(a, b_, 1e-2, 1e-2, name)


@pytest.mark.parametrize("b,h,n,d", [(2, 4, 100, 64), (1, 8, 333, 128)])
def test_gate_combine_matches_oracle(b, h, n, d):
    from native_sparse_attention_pytorch_amd.ops import gate_combine
    g = torch.Generator().manual_seed(b + n)
    c, f, s = (_rand((b, h, n, d), g) for _ in range(3))
    logits = _rand((b, n, 3 * h), g, 2.0)
    do = _rand((b, n, h * d), g)
    ins = [t.float().requires_grad_() for t in (logits, c, f, s)]
    ref = O.gate_combine(*ins)
    (ref * do.float()).sum().backward()
    gins = [t.to(DEV).requires_grad_() for t in (logits, c, f, s)]
    out = gate_combine(*gins)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert_close(out, ref, 2e-2, 1e-2, "gate out")
    for name, a, r in zip(("dlogits", "dc", "df", "ds"), gins, ins):
        _grad_close(a.grad, r.grad, name)


@pytest.mark.parametrize("b,h,n,d,offset,view", [(2, 4, 300, 64, 0, False), (1, 2, 515, 128, 0, True), (1, 4, 64, 64, 40000, False)])
def test_rotary_matches_oracle(b, h, n, d, offset, view):
    """Rotary kernel against the oracle's fp32 restatement, forward and backward, on a contiguous
    tensor and on the 'b n (h d) -> b h n d' view the qkv projection hands over; large positions
    exercise the sine / cosine range reduction.  One bf16 rounding of an O(1) value: 1e-2 abs."""
    from native_sparse_attention_pytorch_amd.ops import rotary
    g = torch.Generator().manual_seed(n + d)
    rot = O.RotaryEmbedding(d)
    if view:
        base = _rand((b, n, h * d), g)
        x = base.view(b, n, h, d).permute(0, 2, 1, 3)
    else:
        x = _rand((b, h, n, d), g)
    do = _rand((b, h, n, d), g)
    xr = x.float().requires_grad_()
    ref = rot.rotate(xr, offset=offset)
    (ref * do.float()).sum().backward()
    xg = x.to(DEV).requires_grad_()
    out = rotary(xg, rot.freqs.to(DEV), offset)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert out.is_contiguous()
    assert_close(out, ref, 1.6e-2 * ref.abs().max().item(), 1e-2, "rotary out")
    _grad_close(xg.grad, xr.grad, "rotary dx")


@pytest.mark.parametrize("b,h,n,d,cbs,st", [(2, 2, 100, 64, 16, 8), (1, 4, 333, 128, 32, 16), (2, 3, 64, 64, 8, 8), (1, 2, 50, 64, 24, 4), (1, 1, 5, 64, 8, 8)])
def test_compress_windows_match_oracle(b, h, n, d, cbs, st):
    """Window gather + position add against the oracle's pad/unfold restatement (itself pinned by a
    brute-force loop), forward and backward (overlap-add), on the strided view the projection gives."""
    from native_sparse_attention_pytorch_amd.ops import compress_windows
    g = torch.Generator().manual_seed(n + cbs)
    base = _rand((b, n, h * d), g)
    x = base.view(b, n, h, d).permute(0, 2, 1, 3)
    pos = _rand((h, cbs, d), g, 0.3)
    L = (n // st) * st
    xr, pr = x.float().requires_grad_(), pos.float().requires_grad_()
    want = O.compress_windows(xr[..., :L, :], cbs, st)
    if want.numel() > 0:
        want = want + pr[None, :, None]
    xg, pg = x.to(DEV).requires_grad_(), pos.to(DEV).requires_grad_()
    got = compress_windows(xg, pg, cbs, st)
    torch.cuda.synchronize()
    assert got.shape == want.shape
    if want.numel() == 0:
        return
    do = _rand(tuple(want.shape), g)
    (want * do.float()).sum().backward()
    (got.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert_close(got, want, 1.6e-2 * want.abs().max().item(), 1e-2, "windows")
    _grad_close(xg.grad, xr.grad, "d tokens")
    _grad_close(pg.grad, pr.grad, "d positions")


def test_topk_long_rows_and_many_selections_bit_exact():
    """Beyond one kernel call (rows over 2048 entries, more than 64 selections - the reference's topk has no limit): per
    segment, then among the segments' winners, 64 at a time.  Bit-exact against the stable sort, exact ties included."""
    from native_sparse_attention_pytorch_amd.ops import importance_topk, topk_op
    g = torch.Generator().manual_seed(5)
    for nb, k in [(4096, 16), (5000, 70), (2049, 3), (300, 100), (6000, 64)]:
        s = torch.rand(2, 1, 20, nb, generator=g)
        s = (s * 64).round() / 64                                # many exact ties
        s[0, 0, :3] = 0.0
        idx, vals, fm = topk_op(s.to(DEV), k, False)
        wv, wi = O.topk_lower_index_first(s, k)
        assert torch.equal(idx.cpu().long(), wi), f"indices differ nb={nb} k={k}"
        assert torch.equal(vals.cpu(), wv) and torch.equal(fm.cpu().bool(), wv > 1e-10)
    # through the padded softmax: the probabilities are torch's own (same formula as the oracle's, on the device)
    logits = torch.randn(1, 2, 30, 4096, generator=g) * 3
    logits[..., :10, 100:] = float("-inf")
    vals, idx, fm = importance_topk(logits.to(DEV), 16)
    probs = O.importance_softmax(logits.to(DEV))
    wv, wi = O.topk_lower_index_first(probs, 16)
    assert torch.equal(idx.long(), wi) and torch.equal(vals, wv) and torch.equal(fm, wv > 1e-10)


def test_select_more_slots_than_one_call_holds():
    """70 selected blocks (one call of the kernels holds 62): the slots go through in groups merged by their log-sum-exp;
    outputs, lse and all gradients against the oracle, which has no such limit (NSA.py:741-819)."""
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    b, hq, hk, n, d, B, S = 1, 4, 2, 1400, 64, 16, 70
    g = torch.Generator().manual_seed(9)
    q, k, v, do = (_rand((b, h, n, d), g, d ** -0.25) for h in (hq, hk, hk, hq))
    from tests.util import causal_random_selection
    idx, msk = causal_random_selection(b, hk, n, B, S, seed=4)
    qr, kr, vr = (t.float().requires_grad_() for t in (q, k, v))
    ref, ref_lse = O.select_attend(qr, kr, vr, idx, msk, B, causal=True, return_lse=True)
    (ref * do.float()).sum().backward()
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    out, lse = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV), return_lse=True)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert_close(out, ref, 2e-2, 1e-2, "out")
    assert_close(lse, ref_lse, 2e-2, 1e-2, "lse")
    _grad_close(qg.grad, qr.grad, "dq")
    _grad_close(kg.grad, kr.grad, "dk")
    _grad_close(vg.grad, vr.grad, "dv")


def test_select_lse_output_carries_gradient():
    """The returned log-sum-exp is differentiable (the merge of slot groups relies on it): a loss on lse alone."""
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    from tests.util import causal_random_selection
    b, hq, hk, n, d, B, S = 1, 4, 2, 300, 64, 16, 3
    g = torch.Generator().manual_seed(13)
    q, k, v = (_rand((b, h, n, d), g, d ** -0.25) for h in (hq, hk, hk))
    w = torch.randn(b, hq, n, generator=g)
    idx, msk = causal_random_selection(b, hk, n, B, S, seed=6)
    qr, kr, vr = (t.float().requires_grad_() for t in (q, k, v))
    _, ref_lse = O.select_attend(qr, kr, vr, idx, msk, B, causal=True, return_lse=True)
    (ref_lse * w).sum().backward()
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    _, lse = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV), return_lse=True)
    (lse * w.to(DEV)).sum().backward()
    torch.cuda.synchronize()
    _grad_close(qg.grad, qr.grad, "dq from lse")
    _grad_close(kg.grad, kr.grad, "dk from lse")
    assert vg.grad is None or float(vg.grad.abs().max()) == 0.0


def test_batch_times_heads_beyond_one_grid():
    """batch * kv heads over 65535 (a grid dimension): the functional entry points cut the batch; every piece equals the same
    rows computed alone."""
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    from native_sparse_attention_pytorch_amd.ops import sliding_attend, compress_attend
    from tests.util import causal_random_selection
    b, hq, hk, n, d, B, S = 66000, 1, 1, 48, 64, 16, 2
    g = torch.Generator().manual_seed(1)
    q = (torch.randn(b, hq, n, d, generator=g) * d ** -0.25).to(torch.bfloat16).to(DEV)
    k, v = q.roll(1, 0), q.roll(2, 0)
    idx, msk = causal_random_selection(1, hk, n, B, S, seed=2)
    idx, msk = idx.expand(b, -1, -1, -1).contiguous().to(DEV), msk.expand(b, -1, -1, -1).contiguous().to(DEV)
    tail = slice(b - 300, b)
    out = native_sparse_attend(q, k, v, B, idx, msk)
    assert torch.equal(out[tail], native_sparse_attend(q[tail], k[tail], v[tail], B, idx[tail], msk[tail]))
    assert torch.equal(out[:100], native_sparse_attend(q[:100], k[:100], v[:100], B, idx[:100], msk[:100]))
    s_out = sliding_attend(q, k, v, 8, causal=True)
    assert torch.equal(s_out[tail], sliding_attend(q[tail], k[tail], v[tail], 8, causal=True))
    ck = k[:, :, :13].contiguous()
    c_out, imp = compress_attend(q, ck, ck, 1, 4, True, sel_block=16, share=True)
    c2, imp2 = compress_attend(q[tail], ck[tail], ck[tail], 1, 4, True, sel_block=16, share=True)
    assert torch.equal(c_out[tail], c2) and torch.equal(imp[tail], imp2)
