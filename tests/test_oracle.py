"""Pins the CPU oracle (oracle/nsa_oracle.py) without the reference package: library
routines (SDPA), brute-force loops on tiny shapes, closed forms and invariants, chosen so
that a dropped term, a wrong sign/index or a transposed operand fails one of them."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import nsa_oracle as O

torch.manual_seed(0)


def sdpa_masked(q, k, v, mask):
    g = q.shape[1] // k.shape[1]
    k = k.repeat_interleave(g, dim=1)
    v = v.repeat_interleave(g, dim=1)
    return F.scaled_dot_product_attention(q, k, v, attn_mask=mask)


# ---------------------------------------------------------------- compress windows

@pytest.mark.parametrize("n,cbs,st", [(12, 4, 2), (10, 5, 2), (8, 4, 4), (9, 8, 2), (0, 4, 2)])
def test_compress_windows_bruteforce(n, cbs, st):
    b, h, d = 2, 3, 5
    L = (n // st) * st
    t = torch.randn(b, h, L, d)
    got = O.compress_windows(t, cbs, st)
    nc = L // st
    assert got.shape == (b, h, nc, cbs, d)
    for w in range(nc):
        for p in range(cbs):
            tok = (w + 1) * st - cbs + p
            want = t[:, :, tok] if tok >= 0 else torch.zeros(b, h, d)
            assert torch.equal(got[:, :, w, p], want)


# ---------------------------------------------------------------------- attend

@pytest.mark.parametrize("hq,hk", [(4, 4), (8, 2)])
def test_attend_matches_sdpa(hq, hk):
    b, n, nc, d, st = 2, 19, 6, 16, 3
    q = torch.randn(b, hq, n, d)
    ck = torch.randn(b, hk, nc + 1, d)
    cv = torch.randn(b, hk, nc + 1, d)
    m = O.compress_mask(n, nc, st)
    out, sim = O.attend(q, ck, cv, mask=m, return_sim=True)
    want = sdpa_masked(q, ck, cv, m)
    assert torch.allclose(out, want, atol=1e-5)
    # head grouping is kv-head-major: query head hq uses kv head hq // G
    g = hq // hk
    for h in range(hq):
        ref = (q[:, h] @ ck[:, h // g].transpose(-1, -2)) * d ** -0.5
        vis = m[None].expand(b, -1, -1)
        assert torch.allclose(sim[:, h][vis], ref[vis], atol=1e-5)
        assert (sim[:, h][~vis] < -1e36).all()


def test_compress_mask_closed_form():
    n, nc, st = 23, 7, 3
    m = O.compress_mask(n, nc, st)
    for i in range(n):
        for c in range(nc + 1):
            assert bool(m[i, c]) == (c * st <= i)      # c counts the memory slot as 0


# --------------------------------------------------------------- importance / top-k

def brute_importance(csim, g, share, st, B):
    """NSA.py:652-695 restated with python loops (fp64)."""
    b, hq, n, ncm = csim.shape
    nc = ncm - 1
    fmax = torch.finfo(csim.dtype).max
    heads = hq // g if share else hq
    npf = B // st
    nb = nc if st == B else nc // npf
    out = torch.zeros(b, heads, n, nb, dtype=torch.float64)
    for bi in range(b):
        for h in range(heads):
            for i in range(n):
                row = []
                for j in range(nb):
                    cs = range(j * npf, (j + 1) * npf) if st != B else [j]
                    hs = range(h * g, (h + 1) * g) if share else [h]
                    val = sum(float(csim[bi, hh, i, 1 + c]) for hh in hs for c in cs) / (len(list(cs)) * len(list(hs)))
                    if st != B and j == i // B:
                        val = -fmax
                    row.append(val)
                row = [-1e3] + row
                mx = max(row)
                e = [math.exp(r - mx) for r in row]
                s = sum(e)
                for j in range(nb):
                    out[bi, h, i, j] = e[j + 1] / s
    return out


@pytest.mark.parametrize("share", [True, False])
@pytest.mark.parametrize("st,B", [(2, 4), (4, 4), (2, 8)])
def test_importance_bruteforce_and_closed_form(share, st, B):
    b, hq, hk, n, d = 1, 4, 2, 21, 8
    g = hq // hk
    nc = n // st
    q = torch.randn(b, hq, n, d)
    ck = torch.randn(b, hk, nc + 1, d)
    cv = torch.randn(b, hk, nc + 1, d)
    _, csim = O.attend(q, ck, cv, mask=O.compress_mask(n, nc, st), return_sim=True)
    got = O.importance_from_csim(csim, 1, g, share, st, B)
    want = brute_importance(csim, g, share, st, B)
    assert got.shape == want.shape
    assert torch.allclose(got.double(), want, atol=1e-6)
    # closed form (causal): only fully completed, strictly earlier blocks score; they form a softmax
    nb = got.shape[-1]
    for i in range(n):
        vis = i // B
        assert (got[:, :, i, vis:] == 0).all()
        if vis > 0:
            assert torch.allclose(got[:, :, i, :vis].sum(-1), torch.ones(b, got.shape[1]), atol=1e-5)


def test_topk_tie_rule_and_values():
    s = torch.tensor([[0.2, 0.5, 0.5, 0.0, 0.0, 0.3]])
    v, i = O.topk_lower_index_first(s, 4)
    assert i.tolist() == [[1, 2, 5, 0]]
    assert torch.equal(v, torch.tensor([[0.5, 0.5, 0.3, 0.2]]))
    x = torch.rand(5, 7, 33)
    v, i = O.topk_lower_index_first(x, 6)
    tv, ti = x.topk(6, dim=-1)
    assert torch.equal(v, tv) and torch.equal(i, ti)      # distinct values: same as torch.topk


# ------------------------------------------------------------ selection attention

def random_selection(b, h, n, B, S, gen, causal=True):
    W = math.ceil(n / B)
    idx = torch.zeros(b, h, n, S, dtype=torch.long)
    msk = torch.zeros(b, h, n, S, dtype=torch.bool)
    for bi in range(b):
        for hh in range(h):
            for i in range(n):
                avail = (i // B) if causal else (n // B)
                k = min(S, avail)
                if k > 0:
                    idx[bi, hh, i, :k] = torch.randperm(avail, generator=gen)[:k]
                    msk[bi, hh, i, :k] = True
    return idx, msk


@pytest.mark.parametrize("n,B,S,hq,hk", [(37, 8, 3, 4, 2), (32, 8, 2, 2, 2), (50, 16, 4, 8, 2)])
@pytest.mark.parametrize("causal", [True, False])
def test_select_attend_equals_dense_mask(n, B, S, hq, hk, causal):
    gen = torch.Generator().manual_seed(1)
    b, d = 2, 16
    q = torch.randn(b, hq, n, d, generator=gen)
    k = torch.randn(b, hk, n, d, generator=gen)
    v = torch.randn(b, hk, n, d, generator=gen)
    idx, msk = random_selection(b, hk, n, B, S, gen, causal)
    if not causal:
        # non-causal rows must attend something: make sure slot 0 is live
        assert msk[..., 0].all() or n // B == 0
    out, lse = O.select_attend(q, k, v, idx, msk, B, causal=causal, return_lse=True, chunk=16)
    W = math.ceil(n / B)
    dm = O.fine_mask(idx, msk, n, B, causal)                     # [b,hk,n,W*B]
    g = hq // hk
    dm = dm.repeat_interleave(g, dim=1)
    kp = F.pad(k, (0, 0, 0, W * B - n))
    vp = F.pad(v, (0, 0, 0, W * B - n))
    want = sdpa_masked(q, kp, vp, dm)
    assert torch.allclose(out, want, atol=1e-5)
    sim = torch.einsum('bhid,bhjd->bhij', q, kp.repeat_interleave(g, dim=1)) * d ** -0.5
    want_lse = torch.logsumexp(sim.masked_fill(~dm, float('-inf')), dim=-1)
    assert torch.allclose(lse, want_lse, atol=1e-5)


def test_select_attend_query_slice():
    gen = torch.Generator().manual_seed(6)
    b, hq, hk, n, d, B, S = 1, 4, 2, 40, 8, 8, 2
    q = torch.randn(b, hq, n, d, generator=gen)
    k = torch.randn(b, hk, n, d, generator=gen)
    v = torch.randn(b, hk, n, d, generator=gen)
    idx, msk = random_selection(b, hk, n, B, S, gen)
    full = O.select_attend(q, k, v, idx, msk, B)
    part = O.select_attend(q[:, :, 19:33], k, v, idx[:, :, 19:33], msk[:, :, 19:33], B, q_offset=19, chunk=5)
    assert torch.allclose(part, full[:, :, 19:33], atol=1e-6)


def test_select_attend_special_cases():
    gen = torch.Generator().manual_seed(2)
    b, hq, hk, n, d, B = 1, 4, 2, 48, 8, 8
    q = torch.randn(b, hq, n, d, generator=gen)
    k = torch.randn(b, hk, n, d, generator=gen)
    v = torch.randn(b, hk, n, d, generator=gen)
    W = n // B
    # every earlier block selected -> full causal attention (textbook)
    idx = torch.arange(W)[None, None, None, :].expand(b, hk, n, W).contiguous()
    msk = idx < (torch.arange(n) // B)[None, None, :, None]
    out = O.select_attend(q, k, v, idx, msk, B, causal=True)
    g = hq // hk
    want = F.scaled_dot_product_attention(q, k.repeat_interleave(g, 1), v.repeat_interleave(g, 1), is_causal=True)
    assert torch.allclose(out, want, atol=1e-5)
    # nothing selected -> block-diagonal causal attention == block_local_attend
    out0 = O.select_attend(q, k, v, idx[..., :0], msk[..., :0], B, causal=True)
    assert torch.allclose(out0, O.block_local_attend(q, k, v, B, True), atol=1e-5)
    out1 = O.select_attend(q, k, v, idx, torch.zeros_like(msk), B, causal=True)
    assert torch.allclose(out1, out0, atol=1e-5)


def test_select_attend_duplicates_and_gates():
    """duplicates count once per slot; a gate multiplies the logits of its slot
    (test_triton_nsa.py:83-96)."""
    b, hq, hk, n, d, B = 1, 2, 1, 16, 4, 4
    gen = torch.Generator().manual_seed(3)
    q = torch.randn(b, hq, n, d, generator=gen)
    k = torch.randn(b, hk, n, d, generator=gen)
    v = torch.randn(b, hk, n, d, generator=gen)
    idx = torch.zeros(b, hk, n, 2, dtype=torch.long)             # block 0 twice
    msk = torch.ones(b, hk, n, 2, dtype=torch.bool)
    gates = torch.rand(b, hk, n, 2, generator=gen) + 0.5
    out = O.select_attend(q, k, v, idx, msk, B, causal=True, gates=gates)
    i = 13
    blk = i // B
    keys = torch.cat((k[0, 0, 0:B] * gates[0, 0, i, 0], k[0, 0, 0:B] * gates[0, 0, i, 1], k[0, 0, blk * B:i + 1]))
    vals = torch.cat((v[0, 0, 0:B], v[0, 0, 0:B], v[0, 0, blk * B:i + 1]))
    for h in range(hq):
        p = torch.softmax((keys @ q[0, h, i]) * d ** -0.5, dim=0)
        assert torch.allclose(out[0, h, i], p @ vals, atol=1e-6)


def test_select_attend_gradcheck_vs_dense():
    gen = torch.Generator().manual_seed(4)
    b, hq, hk, n, d, B, S = 1, 2, 1, 12, 4, 4, 2
    q = torch.randn(b, hq, n, d, generator=gen, dtype=torch.float64, requires_grad=True)
    k = torch.randn(b, hk, n, d, generator=gen, dtype=torch.float64, requires_grad=True)
    v = torch.randn(b, hk, n, d, generator=gen, dtype=torch.float64, requires_grad=True)
    idx, msk = random_selection(b, hk, n, B, S, gen)
    assert torch.autograd.gradcheck(lambda a, b_, c: O.select_attend(a, b_, c, idx, msk, B), (q, k, v), atol=1e-6)


# ----------------------------------------------------------------- sliding attention

@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("n,win", [(33, 4), (20, 64), (17, 1)])
def test_sliding_matches_sdpa(n, win, causal):
    b, hq, hk, d = 2, 4, 2, 8
    q, k, v = torch.randn(b, hq, n, d), torch.randn(b, hk, n, d), torch.randn(b, hk, n, d)
    out = O.sliding_attend(q, k, v, win, causal=causal, chunk=7)
    want = sdpa_masked(q, k, v, O.sliding_mask(n, win, causal))
    assert torch.allclose(out, want, atol=1e-5)
    if causal and win >= n:
        g = hq // hk
        full = F.scaled_dot_product_attention(q, k.repeat_interleave(g, 1), v.repeat_interleave(g, 1), is_causal=True)
        assert torch.allclose(out, full, atol=1e-5)
    # window convention: exactly win+1 keys when causal (NSA.py:524-530)
    assert int(O.sliding_mask(n, win, True)[n - 1].sum()) == min(n, win + 1)


# ----------------------------------------------------------------------------- rotary

def test_rotary_invariants():
    d, n = 16, 11
    r = O.RotaryEmbedding(d)
    assert r.freqs.shape == (d // 2,)
    assert torch.allclose(r.freqs, 10000.0 ** (-torch.arange(0, d, 2).float() / d))
    q, k = torch.randn(1, 1, n, d), torch.randn(1, 1, n, d)
    rq, rk = r.rotate_queries_with_cached_keys(q, k)
    assert torch.allclose(rq[..., 0, :], q[..., 0, :])                       # position 0 is identity
    assert torch.allclose(rq.norm(dim=-1), q.norm(dim=-1), atol=1e-5)        # rotation preserves norm
    # relative property: <R_m x, R_n y> depends on m-n only
    x, y = torch.randn(d), torch.randn(d)
    xs = r.rotate(x.expand(1, 1, n, d))
    ys = r.rotate(y.expand(1, 1, n, d))
    dots = xs[0, 0] @ ys[0, 0].T
    for off in range(-3, 4):
        diag = torch.diagonal(dots, off)
        assert torch.allclose(diag, diag[0].expand_as(diag), atol=1e-4)
    # interleaved pairing: feature pair (0,1) rotates by angle pos*freq[0]
    e0 = torch.zeros(1, 1, 3, d); e0[..., 0] = 1.0
    out = r.rotate(e0)
    assert torch.allclose(out[0, 0, 2, :2], torch.tensor([math.cos(2.0), math.sin(2.0)]), atol=1e-6)
    # single query against cached keys sits at the last position
    rq1, _ = r.rotate_queries_with_cached_keys(q[..., -1:, :], k)
    assert torch.allclose(rq1, rq[..., -1:, :], atol=1e-6)


# ------------------------------------------------------------------------- the module

GRID = [
    # causal, seq, kv_heads, B, cbs, st, S, share
    (False, 31, 8, 4, 4, 2, 2, True),       # BASELINE config 1 (README usage)
    (True, 1, 4, 8, 8, 2, 2, True),
    (True, 4, 8, 16, 4, 4, 0, False),
    (True, 31, 4, 8, 4, 2, 2, False),
    (False, 32, 4, 16, 8, 4, 2, True),
    (True, 120, 4, 32, 8, 4, 2, True),
    (False, 120, 8, 8, 4, 2, 0, True),
    (True, 16, 8, 20, 5, 2, 2, True),       # cbs=5, B=20 as in tests/test_sparse_attn.py:53,67
]


@pytest.mark.parametrize("causal,seq,kvh,B,cbs,st,S,share", GRID)
@pytest.mark.parametrize("diff_topk", [False, True])
def test_module_shape_grid(causal, seq, kvh, B, cbs, st, S, share, diff_topk):
    torch.manual_seed(0)
    m = O.SparseAttentionOracle(512, 64, 8, sliding_window_size=2, compress_block_size=cbs,
                                compress_block_sliding_stride=st, selection_block_size=B,
                                num_selected_blocks=S, kv_heads=kvh, causal=causal,
                                use_diff_topk=diff_topk, query_heads_share_selected_kv=share)
    x = torch.randn(2, seq, 512)
    y = m(x)
    assert y.shape == x.shape and torch.isfinite(y).all()


def test_module_init_invariants_and_gate_closed_form():
    torch.manual_seed(0)
    m = O.SparseAttentionOracle(64, 16, 4, sliding_window_size=4, compress_block_size=4,
                                compress_block_sliding_stride=2, selection_block_size=4,
                                num_selected_blocks=2, kv_heads=2, causal=True)
    sd = m.state_dict()
    for name in ["norm.weight", "rotary_emb.freqs", "to_qkv.weight", "compress_mem_kv", "k_intrablock_positions",
                 "v_intrablock_positions", "k_compress.1.weight", "k_compress.1.bias", "k_compress.3.weight",
                 "k_compress.3.bias", "v_compress.1.weight", "v_compress.3.bias", "to_strategy_combine.0.weight",
                 "to_strategy_combine.0.bias", "combine_heads.weight"]:
        assert name in sd, name
    assert (sd["compress_mem_kv"] == 0).all() and (sd["k_intrablock_positions"] == 0).all()
    assert torch.equal(sd["k_compress.1.weight"], sd["v_compress.1.weight"])
    assert (sd["to_strategy_combine.0.weight"] == 0).all()
    assert sd["to_strategy_combine.0.bias"].tolist() == [-2.0, -2.0, 2.0] * 4
    x = torch.randn(2, 24, 64)
    y, p = m(x, return_parts=True)
    sg = torch.sigmoid(torch.tensor([-2.0, -2.0, 2.0]))
    want = m.combine_heads(O.merge_heads(sg[0] * p["c_out"] + sg[1] * p["f_out"] + sg[2] * p["s_out"]))
    assert torch.allclose(y, want, atol=1e-6)
    # memory slot is zero at init -> its logit is exactly 0
    assert (p["csim"][..., 0] == 0).all()
    # selected blocks: distinct, strictly earlier where live
    idx, vals = p["idx"], p["vals"]
    live = vals > 1e-10
    blk = (torch.arange(24) // 4)[None, None, :, None]
    assert (idx[live] < blk.expand_as(idx)[live]).all()
    srt = idx.sort(dim=-1).values
    assert (srt[..., 1:] != srt[..., :-1]).all()


def test_module_causality():
    torch.manual_seed(0)
    m = O.SparseAttentionOracle(64, 16, 4, sliding_window_size=3, compress_block_size=4,
                                compress_block_sliding_stride=2, selection_block_size=4,
                                num_selected_blocks=2, kv_heads=2, causal=True)
    torch.nn.init.normal_(m.to_strategy_combine[0].weight, std=0.5)
    x = torch.randn(1, 29, 64)
    y = m(x)
    t = 17
    x2 = x.clone()
    x2[:, t:] += torch.randn_like(x2[:, t:])
    y2 = m(x2)
    assert torch.allclose(y[:, :t], y2[:, :t], atol=1e-5)
    assert not torch.allclose(y[:, t:], y2[:, t:], atol=1e-3)


def test_gate_combine_closed_form():
    b, h, n, d = 2, 3, 5, 4
    c, f, s = torch.randn(b, h, n, d), torch.randn(b, h, n, d), torch.randn(b, h, n, d)
    logits = torch.randn(b, n, 3 * h)
    got = O.gate_combine(logits, c, f, s)
    for hh in range(h):
        g = torch.sigmoid(logits[:, :, hh * 3:hh * 3 + 3])                  # column h*3+s
        want = g[..., 0:1] * c[:, hh] + g[..., 1:2] * f[:, hh] + g[..., 2:3] * s[:, hh]
        assert torch.allclose(got[:, :, hh * d:(hh + 1) * d], want, atol=1e-6)


# ------------------------------------------------------------------ decode step (NSA.py:338-547)

@pytest.mark.parametrize("seq_len", (2, 8, 16, 45))
@pytest.mark.parametrize("num_selected_blocks", (0, 2))
@pytest.mark.parametrize("stride", (2, 4))
@pytest.mark.parametrize("block", (8, 16, 20))
@pytest.mark.parametrize("share,kv_heads", ((True, 8), (True, 2), (False, 4)))
def test_decode_steps_equal_parallel_forward(seq_len, num_selected_blocks, stride, block, share, kv_heads):
    """The reference's own criterion for its decode path (tests/test_sparse_attn.py:50-86, same
    grid plus a longer sequence, grouped heads and per-head selection): feeding the tokens one at
    a time through the caches reproduces the parallel forward to 1e-5.  The two code paths share
    no masking or gathering logic, so an off-by-one in either shows up here."""
    torch.manual_seed(seq_len + stride + block)
    m = O.SparseAttentionOracle(dim=64, dim_head=16, heads=8, kv_heads=kv_heads, causal=True, sliding_window_size=2,
                                compress_block_size=5, selection_block_size=block, num_selected_blocks=num_selected_blocks,
                                compress_block_sliding_stride=stride, query_heads_share_selected_kv=share)
    with torch.no_grad():       # away from the symmetric init, but memory slots stay zero as the reference's test has them
        m.to_strategy_combine[0].weight.normal_(std=0.3)
        m.k_intrablock_positions.normal_()
        m.v_intrablock_positions.normal_()
    x = torch.randn(2, seq_len, 64)
    parallel = m(x)
    cache, outs = None, []
    for i in range(seq_len):
        o, cache = m(x[:, i:i + 1], cache=cache, return_cache=True)
        outs.append(o)
    (ck, cv), (run_k, run_v) = cache[1]
    assert cache[0][0].shape[-2] == seq_len and ck.shape[-2] == seq_len // stride
    assert run_k.shape[-2] == (5 - stride) + seq_len % stride
    assert torch.allclose(parallel, torch.cat(outs, dim=1), atol=1e-5)


def test_decode_from_prefill_cache():
    """A prompt through the parallel forward with return_cache, then decode steps: the outputs
    equal the parallel forward of the whole sequence (cache layout of NSA.py:605-619, 863-867)."""
    torch.manual_seed(3)
    m = O.SparseAttentionOracle(dim=64, dim_head=16, heads=4, kv_heads=2, causal=True, sliding_window_size=3,
                                compress_block_size=8, selection_block_size=8, num_selected_blocks=2, compress_block_sliding_stride=4)
    x = torch.randn(1, 37, 64)
    full = m(x)
    for p in (1, 6, 19, 32):
        y, cache = m(x[:, :p], return_cache=True)
        outs = [y]
        for i in range(p, 37):
            o, cache = m(x[:, i:i + 1], cache=cache, return_cache=True)
            outs.append(o)
        assert torch.allclose(full, torch.cat(outs, dim=1), atol=1e-5), p


@pytest.mark.parametrize("block", (4, 8))
def test_transformer_sampling_with_and_without_cache(block):
    """tests/test_sparse_attn.py:88-118: greedy sampling gives the same tokens whether every step
    re-runs the whole prefix or advances the caches."""
    torch.manual_seed(0)
    model = O.TransformerOracle(num_tokens=256, dim=64, depth=2, dim_head=16, heads=4, causal=True,
                                sparse_attn_kwargs=dict(sliding_window_size=16, compress_block_size=4, compress_block_sliding_stride=2,
                                                        selection_block_size=block, num_selected_blocks=2))
    prompt = torch.randint(0, 256, (1, 1))
    a = model.sample(prompt, 48, temperature=0.0, use_cache_kv=False)
    c = model.sample(prompt, 48, temperature=0.0, use_cache_kv=True)
    assert a.shape == (1, 47) and torch.equal(a, c)
