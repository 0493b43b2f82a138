"""Parity of the HIP block-selection attention (through the C ABI) against the CPU oracle.
Tolerances are BASELINE.json's: forward 2e-2 abs / 1e-2 rel in bf16, gradients 5e-2 rel."""

import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import assert_close, assert_grad_close, causal_random_selection

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _inputs(b, hq, hk, n, d, seed):
    g = torch.Generator().manual_seed(seed)
    mk = lambda h: (torch.randn(b, h, n, d, generator=g) * d ** -0.25).to(torch.bfloat16)
    return mk(hq), mk(hk), mk(hk), mk(hq)


def test_mfma_register_layout_selftest():
    from native_sparse_attention_pytorch_amd import _lib
    g = torch.Generator().manual_seed(0)
    A = torch.randn(32, 16, generator=g).to(torch.bfloat16).to(DEV)
    B = torch.randn(16, 32, generator=g).to(torch.bfloat16).to(DEV)
    X = torch.randn(32, 32, generator=g).to(torch.bfloat16).to(DEV)
    Cm = torch.zeros(32, 32, device=DEV)
    T = torch.zeros(32, 32, device=DEV)
    rc = _lib.lib().nsa_selftest_mfma(A.data_ptr(), B.data_ptr(), Cm.data_ptr(), X.data_ptr(), T.data_ptr(),
                                      torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.allclose(Cm.cpu(), A.float().cpu() @ B.float().cpu(), atol=1e-4)
    assert torch.equal(T.cpu(), X.float().cpu())


CASES = [
    # b, hq, hk, n,   d,  B,  S
    (2, 4, 2, 200, 64, 16, 3),       # ragged n, G=2
    (1, 8, 2, 512, 128, 64, 4),      # G=4, d=128
    (1, 4, 4, 300, 64, 32, 5),       # G=1, ragged
    (1, 16, 2, 1024, 64, 64, 16),    # G=8, config-2-like
    (1, 8, 2, 1000, 128, 32, 7),     # ragged, d=128, B=32
    (2, 8, 4, 77, 64, 8, 3),         # 8-key blocks (below the reference Triton path's minimum), ragged
    (1, 4, 1, 250, 128, 8, 6),       # 8-key blocks, G=4, d=128
    (2, 4, 2, 61, 64, 4, 3),         # 4-key blocks: the reference's README / default transformer configuration
    (1, 8, 2, 333, 64, 20, 4),       # 20-key blocks (the reference's inference test grid), ragged
    (1, 4, 2, 200, 128, 48, 2),      # 48 keys: a second, partly filled 32-key tile
    (1, 2, 2, 50, 64, 5, 3),         # odd block size
    (2, 6, 2, 300, 64, 16, 3),       # G=3: not a power of two (padded with zero heads)
    (1, 5, 1, 130, 128, 32, 2),      # G=5
    (1, 8, 2, 1000, 64, 128, 3),     # 128-key blocks: two 64-key sub-blocks per slot, ragged
    (2, 4, 2, 700, 128, 192, 2),     # 192 keys: three sub-blocks
    (1, 4, 1, 400, 64, 96, 2),       # 96 keys: two 48-key sub-blocks
    (2, 4, 2, 200, 32, 16, 3),       # dim_head 32: zero-padded to the kernels' 64
    (1, 4, 2, 300, 96, 32, 2),       # dim_head 96 -> 128
    (1, 2, 1, 100, 40, 8, 2),        # dim_head 40
]


def test_select_more_than_4096_blocks():
    """4125 blocks per sequence: beyond 4096 the index build's list fill runs one wave per chunk of queries instead of four
    (its per-wave position table no longer fits the shared memory a launch may ask for); same checks as the cases below."""
    test_select_fwd_bwd_matches_oracle(1, 2, 1, 33000, 64, 8, 2)


@pytest.mark.parametrize("b,hq,hk,n,d,B,S", CASES)
def test_select_fwd_bwd_matches_oracle(b, hq, hk, n, d, B, S):
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    print(f"case b={b} hq={hq} hk={hk} n={n} d={d} B={B} S={S}", flush=True)
    q, k, v, do = _inputs(b, hq, hk, n, d, seed=n + S)
    idx, msk = causal_random_selection(b, hk, n, B, S, seed=7)

    qr, kr, vr = (t.float().requires_grad_() for t in (q, k, v))
    ref, ref_lse = O.select_attend(qr, kr, vr, idx, msk, B, causal=True, return_lse=True)
    (ref * do.float()).sum().backward()

    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    out, lse = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV), return_lse=True)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()

    assert_close(out, ref, 2e-2, 1e-2, "out")
    assert_close(lse, ref_lse, 1e-2, 1e-3, "lse")
    for name, got, want in (("dq", qg.grad, qr.grad), ("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        assert_grad_close(got, want, name)


def test_select_reference_script_contract():
    """Shapes and input law of test_triton_nsa.py:137-153: ragged n=507, duplicate block ids,
    random slot mask; tolerances of test_triton_nsa.py:189-197."""
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    b, hq, hk, n, d, B, S = 4, 8, 2, 507, 64, 32, 2
    g = torch.Generator().manual_seed(11)
    q, k, v = (torch.randn(b, h, n, d, generator=g).to(torch.bfloat16) for h in (hq, hk, hk))
    idx = torch.randint(0, 2, (b, hk, n, S), generator=g)
    msk = torch.randint(0, 2, (b, hk, n, S), generator=g).bool()
    qr, kr, vr = (t.float().requires_grad_() for t in (q, k, v))
    ref, ref_lse = O.select_attend(qr, kr, vr, idx, msk, B, causal=True, return_lse=True)
    ref.sum().backward()
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    out, lse = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV), return_lse=True)
    out.float().sum().backward()
    torch.cuda.synchronize()
    assert_close(out, ref, 2e-2, 1e-2, "out")
    assert_close(lse, ref_lse, 1e-2, 0, "lse")
    assert_close(vg.grad, vr.grad, 2e-2 * vr.grad.abs().max().item(), 5e-2, "dv")
    assert_close(qg.grad, qr.grad, 2e-2 * qr.grad.abs().max().item(), 5e-2, "dq")
    assert_close(kg.grad, kr.grad, 2e-2 * kr.grad.abs().max().item(), 5e-2, "dk")


def test_select_large_blocks_non_causal_ragged():
    """Blocks of 192 keys (three sub-blocks in the kernels) without the causal own block, ragged sequence: a selected
    last block counts its zero padding past the sequence end, sub-blocks that lie wholly in the padding included."""
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    b, hq, hk, n, d, B, S = 2, 6, 3, 468, 64, 192, 2
    q, k, v, do = _inputs(b, hq, hk, n, d, seed=31)
    g = torch.Generator().manual_seed(32)
    idx = torch.randint(0, 3, (b, hk, n, S), generator=g)
    msk = torch.rand(b, hk, n, S, generator=g) < 0.8
    msk[..., 0] = True
    qr, kr, vr = (t.float().requires_grad_() for t in (q, k, v))
    ref = O.select_attend(qr, kr, vr, idx, msk, B, causal=False)
    (ref * do.float()).sum().backward()
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    out = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV), include_block_causal=False)
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    assert_close(out, ref, 2e-2, 1e-2, "out")
    for name, got, want in (("dq", qg.grad, qr.grad), ("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        assert_grad_close(got, want, name)


def test_select_gate_gradient_matches_oracle():
    """sel_scale (straight-through top-k gates, value 1): its gradient against the oracle's
    gather path with gates multiplying the selected keys (NSA.py:793-797); tolerance of
    test_triton_nsa.py:194 scaled to the gradient's magnitude."""
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    for (b, hq, hk, n, d, B, S) in [(2, 4, 2, 300, 64, 16, 3), (1, 8, 2, 512, 128, 64, 4), (1, 4, 2, 900, 64, 128, 3)]:
        q, k, v, do = _inputs(b, hq, hk, n, d, seed=n)
        idx, msk = causal_random_selection(b, hk, n, B, S, seed=5)
        gr = torch.ones(b, hk, n, S, requires_grad=True)
        qr, kr, vr = (t.float().requires_grad_() for t in (q, k, v))
        ref = O.select_attend(qr, kr, vr, idx, msk, B, causal=True, gates=gr)
        (ref * do.float()).sum().backward()
        gg = torch.ones(b, hk, n, S, device=DEV, requires_grad=True)
        qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
        out = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV), sel_scale=gg)
        (out.float() * do.to(DEV).float()).sum().backward()
        torch.cuda.synchronize()
        want = gr.grad * msk                       # dead slots: the oracle's masked logits carry no gradient either
        assert_grad_close(gg.grad, want, "d sel_scale")
        assert_close(qg.grad, qr.grad, 2e-2 * qr.grad.abs().max().item(), 5e-2, "dq with gates")
        assert (gg.grad.cpu()[~msk] == 0).all()


def test_select_strided_views_and_per_head_selection():
    """q/k/v as 'b n (h d) -> b h n d' views of one projection output (NSA.py:583-585) and
    selection per query head (query_heads_share_selected_kv=False, TRI.py:1961-1962)."""
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    b, hq, hk, n, d, B, S = 2, 4, 2, 256, 64, 16, 4
    g = torch.Generator().manual_seed(5)
    proj = (torch.randn(b, n, (hq + 2 * hk) * d, generator=g) * 0.5).to(torch.bfloat16)
    def views(t):
        q, k, v = t.split((hq * d, hk * d, hk * d), dim=-1)
        sh = lambda x: x.reshape(b, n, -1, d).permute(0, 2, 1, 3)
        return sh(q), sh(k), sh(v)
    idx, msk = causal_random_selection(b, hq, n, B, S, seed=3)
    q, k, v = views(proj.float())
    ref = O.select_attend(q, k, v, idx, msk, B, causal=True)
    qg, kg, vg = views(proj.to(DEV))
    assert not qg.is_contiguous()
    out = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV))
    assert_close(out, ref, 2e-2, 1e-2, "out (strided, per-head selection)")


def test_select_backward_is_bit_reproducible():
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    b, hq, hk, n, d, B, S = 1, 8, 2, 2048, 64, 64, 8
    q, k, v, do = _inputs(b, hq, hk, n, d, seed=1)
    idx, msk = causal_random_selection(b, hk, n, B, S, seed=2)
    grads = []
    for _ in range(2):
        qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
        out = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV))
        (out.float() * do.to(DEV).float()).sum().backward()
        torch.cuda.synchronize()
        grads.append((out.detach().clone(), qg.grad.clone(), kg.grad.clone(), vg.grad.clone()))
    for a, b_ in zip(*grads):
        assert torch.equal(a, b_)


def test_select_full_size_property():
    """BASELINE config 2 size (n=8192, 16/4 heads, d=64, B=64, 15 selected + own block): with
    every earlier block selected where possible the result must equal dense causal attention
    for the first S*B+B tokens, and rows are convex combinations of V everywhere."""
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    b, hq, hk, n, d, B, S = 1, 16, 4, 8192, 64, 64, 15
    q, k, v, _ = _inputs(b, hq, hk, n, d, seed=9)
    idx, msk = causal_random_selection(b, hk, n, B, S, seed=4)
    out, lse = native_sparse_attend(q.to(DEV), k.to(DEV), v.to(DEV), B, idx.to(DEV), msk.to(DEV), return_lse=True)
    m = (S + 1) * B                       # queries below m see their whole causal prefix
    g = hq // hk
    dense = torch.nn.functional.scaled_dot_product_attention(
        q[:, :, :m].float(), k[:, :, :m].float().repeat_interleave(g, 1), v[:, :, :m].float().repeat_interleave(g, 1), is_causal=True)
    assert_close(out[:, :, :m], dense, 2e-2, 1e-2, "dense prefix")
    vmax = v.float().abs().amax(dim=(2,), keepdim=True).repeat_interleave(g, 1)
    assert (out.float().cpu().abs() <= vmax + 1e-2).all()
    assert torch.isfinite(lse).all()
    # brute-force rows for a slice of late queries
    sl = slice(n - 128, n)
    sel_ref = _oracle_rows(q.float(), k.float(), v.float(), idx, msk, B, sl)
    assert_close(out[:, :, sl], sel_ref, 2e-2, 1e-2, "late queries")


def _oracle_rows(q, k, v, idx, msk, B, sl):
    """brute-force (python loops) selection attention for the queries of a slice"""
    import math
    n = q.shape[2]
    out = torch.zeros(q.shape[0], q.shape[1], sl.stop - sl.start, q.shape[3])
    import torch.nn.functional as F
    b, hq, _, d = q.shape
    hk = k.shape[1]
    g = hq // hk
    W = math.ceil(n / B)
    kp = F.pad(k, (0, 0, 0, W * B - n)).reshape(b, hk, W, B, d)
    vp = F.pad(v, (0, 0, 0, W * B - n)).reshape(b, hk, W, B, d)
    for t, i in enumerate(range(sl.start, sl.stop)):
        for bi in range(b):
            for h in range(hk):
                blocks = [int(j) for j, m in zip(idx[bi, h, i], msk[bi, h, i]) if m]
                keys = torch.cat([kp[bi, h, j] for j in blocks] + [k[bi, h, (i // B) * B:i + 1]])
                vals = torch.cat([vp[bi, h, j] for j in blocks] + [v[bi, h, (i // B) * B:i + 1]])
                for gg in range(g):
                    p = torch.softmax((keys @ q[bi, h * g + gg, i]) * d ** -0.5, dim=0)
                    out[bi, h * g + gg, t] = p @ vals
    return out


def test_select_with_sliding_window_output():
    """return_sliding_window_out (TRI.py:1975-1985, test_triton_nsa.py:45-51, 184-189): the second output is causal
    attention over the last block_size + 1 keys; forward and the gradients of the summed loss against the oracle."""
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    b, hq, hk, n, d, B, S = 2, 8, 2, 300, 64, 16, 3
    q, k, v, _ = _inputs(b, hq, hk, n, d, seed=21)
    idx, msk = causal_random_selection(b, hk, n, B, S, seed=22)
    qr, kr, vr = (t.float().requires_grad_() for t in (q, k, v))
    ref, ref_lse = O.select_attend(qr, kr, vr, idx, msk, B, causal=True, return_lse=True)
    ref_s = O.sliding_attend(qr, kr, vr, B, causal=True)
    (ref.sum() + ref_s.sum()).backward()
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    (out, s_out), (lse, s_lse) = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV), return_lse=True, return_sliding_window_out=True)
    (out.float().sum() + s_out.float().sum()).backward()
    torch.cuda.synchronize()
    assert_close(out, ref, 2e-2, 1e-2, "out")
    assert_close(s_out, ref_s, 2e-2, 1e-2, "sliding out")
    assert_close(lse, ref_lse, 1e-2, 1e-3, "lse")
    assert s_lse.shape == lse.shape and torch.isfinite(s_lse).all()
    for name, got, want in (("dq", qg.grad, qr.grad), ("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        assert_grad_close(got, want, name)
