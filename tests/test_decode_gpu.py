"""Single-token decode (NSA.py:338-547) on the HIP path: the two decode attention entry points
through the C ABI against the CPU oracle's attention, then the module's token-by-token decode
against the oracle's decode step and against its own parallel forward.  bf16 inputs, fp32 oracle:
2e-2 abs / 1e-2 rel on outputs."""
import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rand(shape, g, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


RANGE = [
    # b, hq, hk, d, cap, start, count, mem
    (2, 8, 2, 64, 300, 0, 300, 1),
    (1, 16, 4, 128, 2100, 0, 2049, 1),       # compressed keys of a 32k context
    (3, 4, 4, 64, 100, 37, 33, 0),           # sliding window in the middle of the cache
    (2, 8, 1, 128, 64, 0, 1, 0),             # a single key
    (1, 4, 2, 64, 700, 187, 513, 0),
    (2, 6, 2, 64, 90, 0, 70, 3),             # group of 3, three memory slots
    (1, 32, 1, 64, 50, 0, 0, 2),             # memory slots only, 32 heads in one group
]


@pytest.mark.parametrize("b,hq,hk,d,cap,start,count,mem", RANGE)
def test_decode_range_attend_matches_oracle(b, hq, hk, d, cap, start, count, mem):
    from native_sparse_attention_pytorch_amd.ops import decode_range_attend
    print(f"decode range {(b, hq, hk, d, cap, start, count, mem)}", flush=True)
    g = torch.Generator().manual_seed(cap + count)
    q = _rand((b, hq, 1, d), g)
    k, v = _rand((b, hk, cap, d), g), _rand((b, hk, cap, d), g)
    mk, mv = (_rand((hk, mem, d), g), _rand((hk, mem, d), g)) if mem else (None, None)
    kk, vv = k[:, :, start:start + count].float(), v[:, :, start:start + count].float()
    if mem:
        kk = torch.cat((mk.float()[None].expand(b, -1, -1, -1), kk), dim=2)
        vv = torch.cat((mv.float()[None].expand(b, -1, -1, -1), vv), dim=2)
    want, sim = O.attend(q.float(), kk, vv, return_sim=True)
    out, logits = decode_range_attend(q.to(DEV), k.to(DEV), v.to(DEV), start, count,
                                      mk.to(DEV) if mem else None, mv.to(DEV) if mem else None, return_logits=True)
    torch.cuda.synchronize()
    assert out.shape == (b, hq, 1, d)
    assert_close(out, want, 2e-2, 1e-2, "decode range out")
    assert_close(logits, sim[:, :, 0, mem:], 1e-3 * max(1.0, sim.abs().max().item()), 1e-3, "decode logits")


SELECT = [
    # b, hq, hk, d, kv_len, block, S, per_head
    (2, 8, 2, 64, 300, 32, 4, False),
    (1, 16, 4, 128, 2049, 64, 16, False),
    (2, 4, 4, 64, 129, 64, 2, False),        # own block holds one key
    (1, 8, 2, 64, 256, 16, 5, False),        # own block complete
    (2, 8, 2, 64, 333, 32, 3, True),         # every query head selects for itself
    (1, 4, 2, 64, 50, 20, 2, False),         # block size that is no multiple of 16
    (2, 4, 1, 128, 40, 64, 0, False),        # nothing selected: own block only
]


@pytest.mark.parametrize("b,hq,hk,d,kv_len,block,S,per_head", SELECT)
def test_decode_select_attend_matches_oracle(b, hq, hk, d, kv_len, block, S, per_head):
    from native_sparse_attention_pytorch_amd.ops import decode_select_attend
    print(f"decode select {(b, hq, hk, d, kv_len, block, S, per_head)}", flush=True)
    g = torch.Generator().manual_seed(kv_len + S)
    cap = kv_len + 17
    q = _rand((b, hq, 1, d), g)
    k, v = _rand((b, hk, cap, d), g), _rand((b, hk, cap, d), g)
    hs = hq if per_head else hk
    nblk = (kv_len - 1) // block                           # complete earlier blocks
    idx = torch.zeros(b, hs, 1, S, dtype=torch.int64)
    live = torch.zeros(b, hs, 1, S, dtype=torch.bool)
    for bi in range(b):
        for hi in range(hs):
            m = min(S, nblk)
            idx[bi, hi, 0, :m] = torch.randperm(max(nblk, 1), generator=g)[:m]
            live[bi, hi, 0, :m] = torch.rand(m, generator=g) > 0.2
    want = O.select_attend(q.float(), k[:, :, :kv_len].float(), v[:, :, :kv_len].float(), idx, live, block, causal=True, q_offset=kv_len - 1)
    for dt in (torch.int64, torch.int32):
        out = decode_select_attend(q.to(DEV), k.to(DEV), v.to(DEV), kv_len, block, idx.to(dt).to(DEV), live.to(DEV))
        torch.cuda.synchronize()
        assert_close(out, want, 2e-2, 1e-2, f"decode select out {dt}")


def test_rotary_into_cache_slot():
    from native_sparse_attention_pytorch_amd.ops import rotary_into
    g = torch.Generator().manual_seed(5)
    x = _rand((2, 4, 1, 64), g)
    rot = O.RotaryEmbedding(64)
    cache = torch.zeros(2, 4, 40, 64, dtype=torch.bfloat16, device=DEV)
    rotary_into(x.to(DEV), rot.freqs.to(DEV), 17, cache[:, :, 17:18])
    torch.cuda.synchronize()
    assert_close(cache[:, :, 17:18], rot.rotate(x.float(), offset=17), 2e-2, 1e-2, "rotated row")
    assert cache[:, :, :17].abs().max() == 0 and cache[:, :, 18:].abs().max() == 0


def test_decode_prep_rotates_and_fills_cache_rows():
    from native_sparse_attention_pytorch_amd.ops import decode_prep
    g = torch.Generator().manual_seed(6)
    b, hq, hk, d, pos = 3, 8, 2, 128, 301
    qkv = _rand((b, 1, (hq + 2 * hk) * d), g)                     # the projection's layout: heads are views
    q, k, v = (t.view(b, 1, -1, d).permute(0, 2, 1, 3) for t in qkv.split((hq * d, hk * d, hk * d), dim=-1))
    rot = O.RotaryEmbedding(d)
    kc = torch.zeros(b, hk, 400, d, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros_like(kc)
    qkv_d = qkv.to(DEV)
    qd, kd, vd = (t.view(b, 1, -1, d).permute(0, 2, 1, 3) for t in qkv_d.split((hq * d, hk * d, hk * d), dim=-1))
    rq = decode_prep(qd, kd, vd, rot.freqs.to(DEV), pos, kc[:, :, pos:pos + 1], vc[:, :, pos:pos + 1])
    torch.cuda.synchronize()
    assert_close(rq, rot.rotate(q.float(), offset=pos), 3e-2, 1e-2, "rotated queries")
    assert_close(kc[:, :, pos:pos + 1], rot.rotate(k.float(), offset=pos), 3e-2, 1e-2, "rotated key row")
    assert torch.equal(vc[:, :, pos].cpu(), v[:, :, 0])
    kc[:, :, pos] = 0
    vc[:, :, pos] = 0
    assert kc.abs().max() == 0 and vc.abs().max() == 0, "rows other than `pos` were written"


@pytest.mark.parametrize("with_compressed", [True, False])
def test_decode_combine_matches_oracle_gate(with_compressed):
    """Fused merge + sigmoid gate + head merge against the oracle's gate applied to the three
    separately merged branch outputs."""
    from native_sparse_attention_pytorch_amd import ops
    g = torch.Generator().manual_seed(8)
    b, hq, hk, d, n = 2, 8, 2, 64, 500
    q = _rand((b, hq, 1, d), g).to(DEV)
    k, v = _rand((b, hk, n, d), g).to(DEV), _rand((b, hk, n, d), g).to(DEV)
    ck, cv = _rand((b, hk, 60, d), g).to(DEV), _rand((b, hk, 60, d), g).to(DEV)
    mk, mv = _rand((hk, 1, d), g).to(DEV), _rand((hk, 1, d), g).to(DEV)
    idx = torch.tensor([3, 0, 5], dtype=torch.int32, device=DEV).expand(b, hk, 1, 3).contiguous()
    live = torch.ones_like(idx, dtype=torch.bool)
    logits = _rand((b, 1, 3 * hq), g, 2.0).to(DEV)
    outs, parts = [], []
    for merge in (True, False):
        c = ops.decode_range_attend(q, ck, cv, 0, 60, mk, mv, merge=merge) if with_compressed else None
        f = ops.decode_select_attend(q, k, v, n, 64, idx, live, merge=merge)
        s_ = ops.decode_range_attend(q, k, v, n - 33, 33, merge=merge)
        (outs if merge else parts).extend([c, f, s_])
    got = ops.decode_combine(logits, *parts)
    torch.cuda.synchronize()
    c, f, s_ = (torch.zeros(b, hq, 1, d) if t is None else t.float().cpu() for t in outs)
    want = O.gate_combine(logits.float().cpu(), c, f, s_)
    assert got.shape == (b, 1, hq * d)
    assert_close(got, want, 2e-2, 1e-2, "decode combine")


def _pair(seed, **kw):
    from native_sparse_attention_pytorch_amd.sparse_attention import SparseAttention
    torch.manual_seed(seed)
    ref = O.SparseAttentionOracle(**kw)
    with torch.no_grad():
        ref.to_strategy_combine[0].weight.normal_(std=0.05)
        ref.compress_mem_kv.normal_(std=0.5)
        ref.k_intrablock_positions.normal_(std=0.2)
        ref.v_intrablock_positions.normal_(std=0.2)
        for p in ref.parameters():
            p.copy_(p.to(torch.bfloat16).float())
    mod = SparseAttention(**kw)
    mod.load_state_dict(ref.state_dict(), strict=True)
    return ref, mod.to(DEV).to(torch.bfloat16)


DECODE_CONFIGS = [
    dict(dim=256, dim_head=64, heads=8, kv_heads=2, sliding_window_size=24, compress_block_size=16,
         compress_block_sliding_stride=8, selection_block_size=32, num_selected_blocks=3, causal=True),
    dict(dim=128, dim_head=64, heads=4, kv_heads=4, sliding_window_size=5, compress_block_size=4,
         compress_block_sliding_stride=4, selection_block_size=16, num_selected_blocks=2, causal=True),
    dict(dim=256, dim_head=128, heads=4, kv_heads=2, sliding_window_size=16, compress_block_size=24,
         compress_block_sliding_stride=8, selection_block_size=16, num_selected_blocks=2, causal=True,
         query_heads_share_selected_kv=False, num_compressed_mem_kv=2),
]


@pytest.mark.parametrize("ci", range(len(DECODE_CONFIGS)))
@pytest.mark.parametrize("prefill", [1, 70])
def test_module_decode_matches_oracle_decode(ci, prefill):
    """Prefill `prefill` tokens through the parallel forward, then decode token by token; every
    step is compared with the oracle's decode step run under the HIP path's block selection
    (a flipped near-tie in the top-k must not hide or fake a numeric error), and the selections
    themselves must agree almost everywhere."""
    kw = DECODE_CONFIGS[ci]
    print(f"decode module config {ci} prefill {prefill}", flush=True)
    from native_sparse_attention_pytorch_amd import ops
    ref, mod = _pair(10 + ci, **kw)
    n = 150
    g = torch.Generator().manual_seed(ci)
    x = torch.randn(2, n, kw["dim"], generator=g).to(torch.bfloat16)

    with torch.no_grad():
        y, cache = mod(x[:, :prefill].to(DEV), return_cache=True)
        _, rcache = ref(x[:, :prefill].float(), return_cache=True)
    captured = {}
    orig = ops.decode_step
    def spy(*a, **kw_):
        r = orig(*a, **kw_)
        if r[1].shape[-1] > 0:
            captured["sel"] = (r[1].cpu().long(), r[2].cpu())
        return r
    agree = total = 0
    worst = 0.0
    for i in range(prefill, n):
        captured.clear()
        ops.decode_step = spy
        try:
            out, cache = mod(x[:, i:i + 1].to(DEV), cache=cache, return_cache=True)
            torch.cuda.synchronize()
        finally:
            ops.decode_step = orig
        with torch.no_grad():
            own, _ = ref(x[:, i:i + 1].float(), cache=rcache, return_cache=True)           # the oracle's own selection
            want, rcache2 = ref(x[:, i:i + 1].float(), cache=rcache, return_cache=True, selection_override=captured.get("sel"))
        if "sel" in captured:
            nb = rcache[1][0][0].shape[-2] // (kw["selection_block_size"] // kw["compress_block_sliding_stride"])
            assert captured["sel"][0].shape[-1] == min(kw["num_selected_blocks"], nb)
        rcache = rcache2
        assert out.shape == (2, 1, kw["dim"])
        err = (out.float().cpu() - want).abs().max().item()
        worst = max(worst, err / max(want.abs().max().item(), 1e-6))
        assert_close(out, want, 3e-2 * want.abs().max().item(), 2e-2, f"decode step {i}")
        d_own = (own - want).abs().max().item()
        agree += d_own < 1e-4
        total += 1
    assert agree / total > 0.9, f"steps whose selection equals the oracle's own: {agree}/{total}"
    (ck, _), (run_k, _) = cache[1]
    assert cache[0][0].shape[-2] == n and ck.shape[-2] == n // kw["compress_block_sliding_stride"]


def test_module_decode_equals_parallel_forward():
    """The reference's own criterion (tests/test_sparse_attn.py:50-86), at bf16 resolution: the
    token-by-token outputs reproduce the parallel forward of the same module."""
    kw = DECODE_CONFIGS[0]
    _, mod = _pair(3, **kw)
    with torch.no_grad():
        mod.compress_mem_kv.zero_()     # as at init; the reference's decode drops the memory slots before the first compressed key exists
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 200, kw["dim"], generator=g).to(torch.bfloat16).to(DEV)
    with torch.no_grad():
        par = mod(x)
        cache, outs = None, []
        for i in range(200):
            o, cache = mod(x[:, i:i + 1], cache=cache, return_cache=True)
            outs.append(o)
    seq = torch.cat(outs, dim=1)
    torch.cuda.synchronize()
    bad = ((par.float() - seq.float()).abs() > 3e-2 * par.float().abs().max()).any(dim=-1).float().mean().item()
    assert bad < 0.03, f"{bad:.3f} of the tokens differ between decode and parallel forward"


def test_old_cache_stays_valid_when_decoding_branches():
    """Caches are prefixes of growable buffers; decoding twice from the same cache (a branch
    point) must not disturb the first continuation."""
    kw = DECODE_CONFIGS[1]
    _, mod = _pair(4, **kw)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, 40, kw["dim"], generator=g).to(torch.bfloat16).to(DEV)
    with torch.no_grad():
        _, c0 = mod(x[:, :30], return_cache=True)
        _, c1 = mod(x[:, 30:31], cache=c0, return_cache=True)
        a, c2a = mod(x[:, 31:32], cache=c1, return_cache=True)
        keys_a = c2a[0][0].clone()
        b_, c2b = mod(x[:, 35:36], cache=c1, return_cache=True)       # another continuation of c1
        a2, _ = mod(x[:, 31:32], cache=c1, return_cache=True)
    torch.cuda.synchronize()
    assert torch.equal(a, a2)
    assert torch.equal(c2a[0][0], keys_a), "the first continuation's key cache was overwritten"
    assert not torch.equal(c2a[0][0][:, :, -1], c2b[0][0][:, :, -1])


def test_transformer_greedy_sampling_with_and_without_cache():
    """tests/test_sparse_attn.py:88-118 on the HIP path.  bf16 logits can flip an argmax between
    the two code paths, after which the continuations differ legitimately: the first 8 tokens must
    agree, and the cached run must reproduce itself."""
    from native_sparse_attention_pytorch_amd.transformer import Transformer
    torch.manual_seed(0)
    model = Transformer(num_tokens=256, dim=128, depth=2, dim_head=64, heads=4, causal=True,
                        sparse_attn_kwargs=dict(sliding_window_size=16, compress_block_size=8, compress_block_sliding_stride=4,
                                                selection_block_size=16, num_selected_blocks=2)).to(DEV).to(torch.bfloat16)
    prompt = torch.randint(0, 256, (1, 1), device=DEV)
    a = model.sample(prompt, 64, temperature=0., use_cache_kv=False)
    c = model.sample(prompt, 64, temperature=0., use_cache_kv=True)
    c2 = model.sample(prompt, 64, temperature=0., use_cache_kv=True)
    assert a.shape == (1, 63) and torch.equal(c, c2)
    assert torch.equal(a[:, :8], c[:, :8]), (a, c)


@pytest.mark.parametrize("b,hq,hk,nc,npf,share,k", [(2, 8, 2, 37, 4, True, 3), (1, 4, 4, 512, 1, True, 16), (3, 8, 2, 130, 2, False, 5), (1, 16, 1, 2048, 4, True, 16)])
def test_decode_importance_topk_matches_oracle(b, hq, hk, nc, npf, share, k):
    """Fused pooling + padded softmax + top-k of the decode step against the oracle's functions on
    the same logits: indices equal where the probabilities are distinct, values to 1e-5."""
    from native_sparse_attention_pytorch_amd.ops import decode_importance_topk
    g = torch.Generator().manual_seed(nc + k)
    logits = torch.randn(b, hq, nc, generator=g) * 3
    nb = nc // npf
    pooled = logits[..., :nb * npf].reshape(b, hk, hq // hk, nb, npf).mean(dim=-1)
    pooled = pooled.mean(dim=2, keepdim=True) if share else pooled.reshape(b, hq, 1, nb)
    probs = O.importance_softmax(pooled)
    want_v, want_i = O.topk_lower_index_first(probs, k)
    vals, idx, fm = decode_importance_topk(logits.to(DEV), hk, npf, share, k)
    torch.cuda.synchronize()
    assert idx.shape == want_i.shape
    assert_close(vals, want_v, 1e-5, 1e-4, "selected probabilities")
    gap = (want_v[..., :-1] - want_v[..., 1:]).min().item()
    if gap > 1e-6:
        assert torch.equal(idx.cpu().long(), want_i)
    assert torch.equal(fm.cpu(), want_v > 1e-10) or (want_v - 1e-10).abs().min() < 1e-12
