"""The compressed forward that makes the block selection itself (nsa_compress_topk_fwd: no importance logits in memory)
against the two-kernel path on the same inputs - the logits written out by nsa_dense_fwd, then nsa_topk - and, through
that, against the oracle (NSA.py:652-721): same attention output bit for bit (the same MFMA walk), same slot mask, same
block indices in every live slot, in the same order; exact ties go to the lower block index."""
import pytest
import torch

from oracle import nsa_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rand(shape, g, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def _both(q, ck, cv, mem, st, causal, B, k):
    from native_sparse_attention_pytorch_amd import ops
    assert ops.compress_topk_supported(q, ck, mem, st, B, k, True)
    out1, idx1, fm1 = ops.compress_attend_topk(q, ck, cv, mem, st, causal, B, k)
    out2, imp = ops.compress_attend(q, ck, cv, mem, st, causal, sel_block=B, share=True)
    vals2, idx2, fm2 = ops.importance_topk(imp.contiguous(), k)
    torch.cuda.synchronize()
    return (out1, idx1, fm1), (out2, idx2, fm2, vals2, imp)


CASES = [
    # b, hq, hk, n, d, st, B, mem, causal, k
    (1, 8, 2, 2100, 128, 16, 64, 1, True, 16),       # config-4 geometry (group 4, 4 compressed keys per block), ragged end
    (2, 16, 4, 1024, 64, 16, 64, 1, True, 16),       # config-3 geometry
    (2, 8, 4, 1024, 64, 8, 16, 1, True, 4),          # config-5 geometry: group 2, 2 keys per block, 4 selected
    (1, 8, 1, 700, 64, 4, 4, 2, True, 16),           # group 8, stride == block (64 candidates per key tile), two memory slots
    (1, 4, 2, 900, 64, 2, 16, 1, True, 7),           # 8 keys per block
    (1, 4, 2, 1500, 128, 2, 32, 1, True, 16),        # 16 keys per block
    (1, 4, 1, 2000, 64, 2, 64, 1, True, 5),          # 32 keys per block
    (1, 8, 2, 777, 64, 8, 32, 1, False, 16),         # non-causal: every block but the query's own
    (1, 4, 2, 300, 64, 16, 16, 1, False, 8),         # non-causal, stride == block: own block selectable as well
    (1, 16, 1, 333, 128, 16, 64, 1, True, 3),        # group 16: two queries per wave tile; fewer blocks than a full list
    (1, 64, 2, 200, 64, 4, 16, 1, True, 6),          # group 32: one query per wave tile
]


@pytest.mark.parametrize("b,hq,hk,n,d,st,B,mem,causal,k", CASES)
def test_fused_selection_equals_logits_then_topk(b, hq, hk, n, d, st, B, mem, causal, k):
    print(f"fused top-k b={b} hq={hq} hk={hk} n={n} d={d} st={st} B={B} mem={mem} causal={causal} k={k}", flush=True)
    g = torch.Generator().manual_seed(n + d + st)
    nc = n // st
    q = _rand((b, hq, n, d), g, d ** -0.25).to(DEV)
    ck, cv = _rand((b, hk, mem + nc, d), g, d ** -0.25).to(DEV), _rand((b, hk, mem + nc, d), g).to(DEV)
    (out1, idx1, fm1), (out2, idx2, fm2, vals2, imp) = _both(q, ck, cv, mem, st, causal, B, k)
    assert torch.equal(out1, out2), "attention output differs between the two forward variants"
    assert torch.equal(fm1, fm2), f"slot mask differs in {(fm1 != fm2).sum().item()} slots"
    live = fm2
    assert live.any()
    assert torch.equal(idx1[live], idx2[live]), f"{(idx1[live] != idx2[live]).sum().item()} live slots name another block"
    nb = imp.shape[-1]
    assert int(idx1.min()) >= 0 and int(idx1.max()) < nb


def test_fused_selection_matches_oracle_selection():
    """Against the oracle directly: its importance scores from its own compressed attention logits, stable top-k."""
    b, hq, hk, n, d, st, B, mem, k = 1, 8, 2, 600, 64, 4, 16, 1, 6
    g = torch.Generator().manual_seed(3)
    nc = n // st
    q = _rand((b, hq, n, d), g, d ** -0.25)
    ck, cv = _rand((b, hk, mem + nc, d), g, d ** -0.25), _rand((b, hk, mem + nc, d), g)
    from native_sparse_attention_pytorch_amd import ops
    out, idx, fm = ops.compress_attend_topk(q.to(DEV), ck.to(DEV), cv.to(DEV), mem, st, True, B, k)
    want_out, csim = O.attend(q.float(), ck.float(), cv.float(), mask=O.compress_mask(n, nc, st, mem, True), return_sim=True)
    scores = O.importance_softmax(O.importance_logits(csim, mem, hq // hk, True, st, B))
    vals, widx = O.topk_lower_index_first(scores, k)
    wlive = vals > 1e-10
    assert (out.float().cpu() - want_out).abs().max() < 2e-2
    # bf16 logits against fp32 logits: near-ties may swap; the live sets must agree almost everywhere and the masks exactly in count
    fm, idx = fm.cpu(), idx.cpu().long()
    assert torch.equal(fm.sum(-1), wlive.sum(-1)), "number of live slots per query differs from the oracle's"
    agree = total = 0
    for a, la, w, lw in zip(idx.flatten(0, 2), fm.flatten(0, 2), widx.flatten(0, 2), wlive.flatten(0, 2)):
        sa, sw = set(a[la].tolist()), set(w[lw].tolist())
        agree += len(sa & sw)
        total += max(len(sa), len(sw))
    assert agree / total > 0.97, f"selected-block agreement {agree}/{total}"


def test_fused_selection_exact_ties_take_the_lower_block():
    """Blocks whose compressed keys are bit-for-bit copies of an earlier block's have bit-equal logits for every query: among
    equals the lower block index is selected first, and the order of the outputs shows it."""
    b, hq, hk, n, d, st, B, mem, k = 1, 4, 1, 1024, 64, 16, 64, 1, 16
    npf = B // st
    g = torch.Generator().manual_seed(11)
    nc = n // st
    q = _rand((b, hq, n, d), g, d ** -0.25)
    ck, cv = _rand((b, hk, mem + nc, d), g, d ** -0.25), _rand((b, hk, mem + nc, d), g)
    blk = lambda j: slice(mem + j * npf, mem + (j + 1) * npf)
    for dst, src in ((5, 2), (9, 2), (12, 7), (13, 7), (14, 7), (3, 0)):
        ck[:, :, blk(dst)] = ck[:, :, blk(src)]
    q, ck, cv = q.to(DEV), ck.to(DEV), cv.to(DEV)
    (out1, idx1, fm1), (out2, idx2, fm2, vals2, imp) = _both(q, ck, cv, mem, st, True, B, k)
    # (for the queries that see both blocks completely)
    assert torch.equal(imp[..., 6 * B:, 5], imp[..., 6 * B:, 2]) and torch.equal(imp[..., 14 * B:, 13], imp[..., 14 * B:, 7]), "the copies must tie exactly"
    assert torch.equal(fm1, fm2) and torch.equal(idx1[fm2], idx2[fm2])
    # in the last query's list every copy comes right after its original, lower index first
    last = idx1[0, 0, n - 1].tolist()
    for group in ((2, 5, 9), (7, 12, 13, 14), (0, 3)):
        pos = [last.index(j) for j in group]
        assert pos == list(range(pos[0], pos[0] + len(group))), (group, last)


def test_fused_selection_refuses_what_it_does_not_serve():
    from native_sparse_attention_pytorch_amd import ops
    q = torch.zeros(1, 4, 256, 64, dtype=torch.bfloat16, device=DEV)
    ck = torch.zeros(1, 4, 17, 64, dtype=torch.bfloat16, device=DEV)          # groups of one head
    assert not ops.compress_topk_supported(q, ck, 1, 16, 64, 4, True)
    with pytest.raises(RuntimeError):
        ops.compress_topk_fwd(q, ck, ck, True, 16, 1, 64, 4, 0.125)
    ck2 = torch.zeros(1, 2, 65, 64, dtype=torch.bfloat16, device=DEV)
    assert not ops.compress_topk_supported(q, ck2, 1, 4, 16, 17, True)        # more than 16 selections
    assert not ops.compress_topk_supported(q, ck2, 1, 4, 16, 4, False)        # per-head selection
    assert ops.compress_topk_supported(q, ck2, 1, 4, 16, 16, True)


def test_fused_selection_backward_equals_the_two_kernel_path():
    """The output of the fused forward is differentiable like compress_attend's (the selection carries no gradient): same
    saved output and log-sum-exp, same backward kernels, so the gradients of q and the compressed keys / values are equal bit
    for bit."""
    from native_sparse_attention_pytorch_amd import ops
    b, hq, hk, n, d, st, B, mem, k = 2, 8, 2, 1100, 64, 8, 32, 1, 8
    g = torch.Generator().manual_seed(21)
    nc = n // st
    mk = lambda *s, sc=1.0: (torch.randn(*s, generator=g) * sc).to(torch.bfloat16).to(DEV)
    q, ck, cv, do = mk(b, hq, n, d, sc=d ** -0.25), mk(b, hk, mem + nc, d, sc=d ** -0.25), mk(b, hk, mem + nc, d), mk(b, hq, n, d)
    grads = []
    for fused in (True, False):
        q1, ck1, cv1 = (t.clone().requires_grad_() for t in (q, ck, cv))
        out = ops.compress_attend_topk(q1, ck1, cv1, mem, st, True, B, k)[0] if fused else ops.compress_attend(q1, ck1, cv1, mem, st, True, sel_block=B, share=True)[0]
        out.backward(do)
        grads.append((q1.grad, ck1.grad, cv1.grad))
    torch.cuda.synchronize()
    for name, a, b_ in zip(("dq", "dck", "dcv"), *grads):
        assert a is not None and torch.isfinite(a).all(), name
        assert torch.equal(a, b_), f"{name}: {(a.float() - b_.float()).abs().max().item()}"
