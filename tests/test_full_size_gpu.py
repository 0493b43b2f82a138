"""The three attention branches at the headline size (sequence 32768, 32 query / 8 kv heads,
dim_head 128, selection block 64, 15 selected + own block, compress stride 16) against the CPU
oracle.  The oracle cannot run the whole problem in seconds, so each test arranges that a part
of it is complete in itself:
  * selection: the upstream gradient is non-zero only for the queries of a few blocks, so the
    oracle run on just those queries yields every gradient of the full problem (dK/dV of all
    blocks included) and the remaining dQ rows must be exactly zero;
  * compressed and sliding: heads are independent, so the oracle runs one kv head (4 query
    heads) of the full-length problem.
Tolerances are the same as for the small cases: forward 2e-2 abs / 1e-2 rel, gradients 5e-2 rel."""
import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import assert_close, assert_grad_close, causal_random_selection

pytestmark = pytest.mark.gpu
DEV = "cuda"

B_, HQ, HK, N, D = 1, 32, 8, 32768, 128
G = HQ // HK
BLOCK, S, STRIDE = 64, 15, 16


def _rand(shape, g, scale):
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def _grad_close(got, want, name):
    assert_grad_close(got, want, name)


def test_selection_32k_forward_and_backward():
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    g = torch.Generator().manual_seed(32)
    q, k, v = _rand((B_, HQ, N, D), g, D ** -0.25), _rand((B_, HK, N, D), g, D ** -0.25), _rand((B_, HK, N, D), g, 1.0)
    idx, msk = causal_random_selection(B_, HK, N, BLOCK, S, seed=33)
    blocks = [0, 9, 16, 201, 388, 510, 511]            # query blocks that carry upstream gradient
    do = torch.zeros(B_, HQ, N, D, dtype=torch.bfloat16)
    for w in blocks:
        do[:, :, w * BLOCK:(w + 1) * BLOCK] = _rand((B_, HQ, BLOCK, D), g, 1.0)
    print("selection 32k: oracle on", len(blocks), "query blocks", flush=True)

    kr, vr = k.float().requires_grad_(), v.float().requires_grad_()
    loss, ref = 0.0, {}
    for w in blocks:
        sl = slice(w * BLOCK, (w + 1) * BLOCK)
        qr = q[:, :, sl].float().requires_grad_()
        o, lse = O.select_attend(qr, kr, vr, idx[:, :, sl], msk[:, :, sl], BLOCK, causal=True, return_lse=True, q_offset=w * BLOCK)
        loss = loss + (o * do[:, :, sl].float()).sum()
        ref[w] = (qr, o.detach(), lse.detach())
    loss.backward()

    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    out, lse = native_sparse_attend(qg, kg, vg, BLOCK, idx.to(DEV), msk.to(DEV), return_lse=True)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()

    dq = qg.grad.cpu()
    live = torch.zeros(N, dtype=torch.bool)
    dq_scale = max(r[0].grad.abs().max().item() for r in ref.values())
    for w in blocks:
        sl = slice(w * BLOCK, (w + 1) * BLOCK)
        live[sl] = True
        qr, o, l = ref[w]
        assert_close(out[:, :, sl], o, 2e-2, 1e-2, f"out, query block {w}")
        assert_close(lse[:, :, sl], l, 1e-2, 1e-3, f"lse, query block {w}")
        assert_close(dq[:, :, sl], qr.grad, 2e-2 * dq_scale, 5e-2, f"dq, query block {w}")
    assert (dq[:, :, ~live] == 0).all(), "queries without upstream gradient must get dq == 0"
    _grad_close(kg.grad, kr.grad, "dk (all 512 blocks)")
    _grad_close(vg.grad, vr.grad, "dv (all 512 blocks)")
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()


def test_compressed_branch_32k_one_kv_head_and_topk():
    from native_sparse_attention_pytorch_amd.ops import compress_attend, importance_topk
    g = torch.Generator().manual_seed(34)
    mem, nc = 1, N // STRIDE
    q = _rand((B_, HQ, N, D), g, D ** -0.25)
    ck, cv = _rand((B_, HK, mem + nc, D), g, D ** -0.25), _rand((B_, HK, mem + nc, D), g, 1.0)
    do = _rand((B_, HQ, N, D), g, 1.0)
    hk = 5
    hs = slice(hk * G, (hk + 1) * G)
    print("compressed 32k: oracle on kv head", hk, flush=True)

    qr, kr, vr = q[:, hs].float().requires_grad_(), ck[:, hk:hk + 1].float().requires_grad_(), cv[:, hk:hk + 1].float().requires_grad_()
    ref, csim = O.attend(qr, kr, vr, mask=O.compress_mask(N, nc, STRIDE, mem, True), return_sim=True)
    (ref * do[:, hs].float()).sum().backward()
    want_imp = O.importance_logits(csim.detach(), mem, G, True, STRIDE, BLOCK)
    del csim

    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, ck, cv))
    out, imp = compress_attend(qg, kg, vg, mem, STRIDE, True, sel_block=BLOCK, share=True)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert_close(out[:, hs], ref, 2e-2, 1e-2, "compressed out")
    _grad_close(qg.grad[:, hs], qr.grad, "dq")
    _grad_close(kg.grad[:, hk:hk + 1], kr.grad, "dck")
    _grad_close(vg.grad[:, hk:hk + 1], vr.grad, "dcv")

    got_imp = imp[:, hk:hk + 1].cpu()
    dead = want_imp < -1e30
    assert torch.equal(torch.isinf(got_imp) & (got_imp < 0), dead), "set of unselectable blocks differs"
    assert_close(got_imp[~dead], want_imp[~dead], 2e-3, 1e-3, "importance logits")

    # top-k over all heads: values against the oracle's softmax + stable sort of the same logits (one head),
    # structural properties everywhere
    vals, idx, fm = importance_topk(imp, S)
    vals, idx, fm = vals.cpu(), idx.cpu().long(), fm.cpu().bool()
    p = O.importance_softmax(got_imp.masked_fill(torch.isinf(got_imp), -3.4e37))
    wv1, wi1 = O.topk_lower_index_first(p, S + 1)              # one more, to see a near-tie at the cut
    wv, wi = wv1[..., :S], wi1[..., :S]
    assert_close(vals[:, hk:hk + 1], wv, 1e-6, 1e-4, "top-k values")
    gap = (wv1[..., :-1] - wv1[..., 1:]) > 1e-4 * wv1[..., :-1].clamp_min(1e-30)   # the kernel's fast exp is good to ~1e-6 relative
    clear = gap.clone()                                        # slot s is clear of slot s+1 ...
    clear[..., 1:] &= gap[..., :-1]                            # ... and of slot s-1
    sel = clear & (wv > 1e-10)
    nbad = int((idx[:, hk:hk + 1][sel] != wi[sel]).sum())
    assert nbad == 0, f"{nbad} of {int(sel.sum())} selected blocks differ where the order is not a near-tie"
    assert sel.float().mean() > 0.5
    assert torch.equal(fm, vals > 1e-10)
    assert (vals[..., :-1] >= vals[..., 1:]).all(), "values must come out in descending order"
    own = (torch.arange(N) // BLOCK)[None, None, :, None]
    assert (idx[fm] < own.expand_as(idx)[fm]).all(), "a live slot may only name a completed earlier block"
    srt = idx.masked_fill(~fm, -1).sort(dim=-1).values
    dup = (srt[..., 1:] == srt[..., :-1]) & (srt[..., 1:] >= 0)
    assert not dup.any(), "a block was selected twice"
    # a query in block w has w candidate blocks: min(w, S) of them are selected unless a probability underflows
    full = fm[:, :, S * BLOCK:].float().mean().item()
    assert full > 0.99, full


def test_sliding_branch_32k_one_kv_head():
    from native_sparse_attention_pytorch_amd.ops import sliding_attend
    win = 512
    g = torch.Generator().manual_seed(35)
    q, k, v = _rand((B_, HQ, N, D), g, D ** -0.25), _rand((B_, HK, N, D), g, D ** -0.25), _rand((B_, HK, N, D), g, 1.0)
    do = _rand((B_, HQ, N, D), g, 1.0)
    hk = 2
    hs = slice(hk * G, (hk + 1) * G)
    print("sliding 32k: oracle on kv head", hk, flush=True)
    qr, kr, vr = q[:, hs].float().requires_grad_(), k[:, hk:hk + 1].float().requires_grad_(), v[:, hk:hk + 1].float().requires_grad_()
    ref = O.sliding_attend(qr, kr, vr, win, causal=True)
    (ref * do[:, hs].float()).sum().backward()
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    out = sliding_attend(qg, kg, vg, win, causal=True)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert_close(out[:, hs], ref, 2e-2, 1e-2, "sliding out")
    _grad_close(qg.grad[:, hs], qr.grad, "dq")
    _grad_close(kg.grad[:, hk:hk + 1], kr.grad, "dk")
    _grad_close(vg.grad[:, hk:hk + 1], vr.grad, "dv")
