"""DecodeSession (decode steps replayed from a captured HIP graph, lengths read from device memory)
against the module's eager decode step, replay by replay: the outputs within the bf16 forward
tolerance (the two split the key range differently), the caches bit-equal."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"

CONFIGS = [
    # dim, d, heads, kv, win, cbs, st, B, S, share, prefill, steps
    (256, 64, 4, 2, 16, 8, 4, 8, 2, True, 37, 45),
    (256, 128, 2, 1, 32, 16, 8, 16, 3, True, 70, 40),
    (256, 64, 4, 2, 8, 8, 8, 8, 4, False, 21, 30),        # stride == block, selection per query head
    (128, 64, 2, 2, 16, 8, 4, 8, 2, True, 2, 40),         # starts before the first compressed key exists
    (192, 64, 6, 2, 16, 8, 4, 8, 2, True, 30, 30),        # group of 3 query heads per kv head
    (128, 64, 4, 2, 16, 32, 16, 128, 2, True, 300, 30),   # 128-token selection blocks
    (128, 64, 2, 1, 4, 5, 4, 20, 2, True, 47, 40),        # compress block 5, selection block 20 (5 compressed keys per block)
    (128, 32, 4, 2, 16, 8, 4, 8, 2, True, 37, 30),        # head dimensions the kernels are not compiled for: zero-padded buffers
    (192, 96, 2, 1, 16, 8, 4, 16, 2, True, 40, 30),
]


@pytest.mark.parametrize("cfg", CONFIGS)
def test_graph_decode_matches_eager_decode(cfg):
    from native_sparse_attention_pytorch_amd import SparseAttention
    from native_sparse_attention_pytorch_amd.decode_session import DecodeSession
    from tests.util import assert_close
    dim, d, heads, kv, win, cbs, st, B, S, share, n0, steps = cfg
    print("graph decode", cfg, flush=True)
    torch.manual_seed(sum(cfg[:9]))
    m = SparseAttention(dim=dim, dim_head=d, heads=heads, kv_heads=kv, sliding_window_size=win, compress_block_size=cbs,
                        compress_block_sliding_stride=st, selection_block_size=B, num_selected_blocks=S, causal=True,
                        query_heads_share_selected_kv=share).to(DEV).bfloat16()
    with torch.no_grad():                                          # the gate and memory parameters start at constants
        m.compress_mem_kv.normal_(std=0.5)
        m.k_intrablock_positions.normal_(std=0.2)
        m.v_intrablock_positions.normal_(std=0.2)
        m.to_strategy_combine[0].weight.normal_(std=0.05)
    b = 2
    xs = torch.randn(b, n0 + steps, dim, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        _, cache = m(xs[:, :n0], return_cache=True)
        full = m(xs)                                               # the parallel forward over the whole sequence
    sess = DecodeSession(m, cache, max_len=n0 + steps + 5)
    far = 0
    for i in range(steps):
        x = xs[:, n0 + i:n0 + i + 1]
        with torch.no_grad():
            want, cache = m(x, cache=cache, return_cache=True)
        got = sess.step(x)
        torch.cuda.synchronize()
        assert_close(got, want, 2e-2, 1e-2, f"step {i}")
        # decode against the parallel forward (tests/test_sparse_attn.py:50-86): equal up to bf16 rounding, except where a
        # near-tie selects another block or, before the first compressed key exists, the reference's decode step drops the
        # memory slots the parallel forward attends (NSA.py:401) - those steps are skipped
        if cache[1][0][0].shape[-2] > 1:
            err = (want.float() - full[:, n0 + i:n0 + i + 1].float()).abs().max().item()
            far += err > 3e-2 * max(1.0, full.float().abs().max().item())
    assert far <= steps // 10, f"{far} of {steps} decode steps differ from the parallel forward"
    (k, v), ((ck, cv), (rk, rv)) = sess.cache()
    (k2, v2), ((ck2, cv2), (rk2, rv2)) = cache
    assert torch.equal(k, k2) and torch.equal(v, v2)
    assert ck.shape == ck2.shape and torch.equal(ck, ck2.to(ck.dtype)) and torch.equal(cv, cv2.to(cv.dtype))
    assert rk.shape == rk2.shape and torch.equal(rk, rk2.to(rk.dtype)) and torch.equal(rv, rv2.to(rv.dtype))
    # and back: the module continues from the session's caches
    x = torch.randn(b, 1, dim, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        a, _ = m(x, cache=sess.cache(), return_cache=True)
        bb, _ = m(x, cache=cache, return_cache=True)
    assert torch.equal(a, bb)
    # a session can also start from caches that went through the module's decode steps (padded rows for odd head sizes)
    sess2 = DecodeSession(m, cache, max_len=n0 + steps + 5)
    assert torch.equal(sess2.step(x), sess.step(x))


def test_graph_decode_capacity_is_enforced():
    from native_sparse_attention_pytorch_amd import SparseAttention
    from native_sparse_attention_pytorch_amd.decode_session import DecodeSession
    torch.manual_seed(0)
    m = SparseAttention(dim=128, dim_head=64, heads=2, kv_heads=1, sliding_window_size=8, compress_block_size=8,
                        compress_block_sliding_stride=4, selection_block_size=8, num_selected_blocks=2, causal=True).to(DEV).bfloat16()
    x = torch.randn(1, 12, 128, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        _, cache = m(x, return_cache=True)
    with pytest.raises(ValueError):
        DecodeSession(m, cache, max_len=12)
    sess = DecodeSession(m, cache, max_len=14)
    sess.step(x[:, :1])
    sess.step(x[:, :1])
    with pytest.raises(RuntimeError):
        sess.step(x[:, :1])
    # a caller that replays the graph anyway finds the device-side counters clamped to the capacity: nothing is written
    k_before, v_before = sess.K.clone(), sess.V.clone()
    for _ in range(3):
        sess.graphs[0].replay()
    torch.cuda.synchronize()
    assert torch.equal(sess.K, k_before) and torch.equal(sess.V, v_before)
    assert int(sess.state[0]) == 17


def test_graph_decode_when_prefill_fills_every_compressed_row():
    """A prompt whose compressed keys already fill the compressed caches to their capacity (64 tokens, stride 8,
    room for 66: eight rows, a multiple of the row padding): the capture warm-up still writes one window, which must
    land in the spare row, and the remaining steps run and agree with the eager decode."""
    from native_sparse_attention_pytorch_amd import SparseAttention
    from native_sparse_attention_pytorch_amd.decode_session import DecodeSession
    from tests.util import assert_close
    torch.manual_seed(2)
    m = SparseAttention(dim=128, dim_head=64, heads=2, kv_heads=1, sliding_window_size=8, compress_block_size=16,
                        compress_block_sliding_stride=8, selection_block_size=16, num_selected_blocks=2, causal=True).to(DEV).bfloat16()
    xs = torch.randn(1, 66, 128, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        _, cache = m(xs[:, :64], return_cache=True)
    sess = DecodeSession(m, cache, max_len=66)
    assert sess.nc == sess.max_nc == 8 and sess.CK.shape[2] == 9
    for i in (64, 65):
        with torch.no_grad():
            want, cache = m(xs[:, i:i + 1], cache=cache, return_cache=True)
        got = sess.step(xs[:, i:i + 1])
        torch.cuda.synchronize()
        assert_close(got, want, 2e-2, 1e-2, f"step {i}")
    assert torch.equal(sess.cache()[1][0][0], cache[1][0][0][:, :, :8].to(torch.bfloat16))


def test_transformer_graph_decode_matches_cached_decode():
    """Whole-model graph replay (embedding, 3 layers, logits) against the model's eager cached decode on the same token
    sequence, replay by replay, across compression steps; then sampling through the graph."""
    from native_sparse_attention_pytorch_amd.transformer import Transformer
    from native_sparse_attention_pytorch_amd.decode_session import TransformerDecodeSession
    from tests.util import assert_close
    torch.manual_seed(5)
    model = Transformer(num_tokens=256, dim=128, depth=3, dim_head=64, heads=4, kv_heads=2,
                        sparse_attn_kwargs=dict(sliding_window_size=16, compress_block_size=8, compress_block_sliding_stride=4,
                                                selection_block_size=8, num_selected_blocks=2)).to(DEV).bfloat16()
    ids = torch.randint(0, 256, (2, 70), device=DEV)
    n0 = 19
    with torch.no_grad():
        _, caches = model(ids[:, :n0], return_cache=True)
    sess = TransformerDecodeSession(model, caches, max_len=70)
    for i in range(n0, 70):
        with torch.no_grad():
            want, caches = model(ids[:, :i + 1], cache=caches, return_cache=True)
        got = sess.step(ids[:, i])
        torch.cuda.synchronize()
        assert_close(got, want, 5e-2, 2e-2, f"logits at position {i}")
    assert sess.pos == 70
    with pytest.raises(RuntimeError):
        sess.step(ids[:, 0])

    prompt = ids[:, :12]
    a = model.sample(prompt, 40, temperature=0., use_cache_kv=True)
    b = model.sample(prompt, 40, temperature=0., use_cache_kv=True, use_graph=True)
    assert a.shape == b.shape == (2, 28) and b.dtype == torch.long
    assert torch.equal(a[:, 0], b[:, 0])                     # the first new token comes from the same prefill
    assert (a == b).float().mean() > 0.5                     # greedy paths agree until a near-tie flips a token


def test_graph_decode_with_custom_strategy_network():
    """A caller-supplied strategy_combine_mlp (NSA.py:315-327) is not a plain projection: the session then runs it as it is
    instead of folding it into the qkv GEMM."""
    from torch import nn
    from native_sparse_attention_pytorch_amd import SparseAttention
    from native_sparse_attention_pytorch_amd.decode_session import DecodeSession
    from tests.util import assert_close
    torch.manual_seed(11)
    dim, heads = 128, 4
    m = SparseAttention(dim=dim, dim_head=64, heads=heads, kv_heads=2, sliding_window_size=8, compress_block_size=8,
                        compress_block_sliding_stride=4, selection_block_size=8, num_selected_blocks=2, causal=True,
                        strategy_combine_mlp=nn.Sequential(nn.Linear(dim, 32), nn.ReLU(), nn.Linear(32, 3 * heads))).to(DEV).bfloat16()
    xs = torch.randn(2, 40, dim, device=DEV, dtype=torch.bfloat16)
    with torch.no_grad():
        _, cache = m(xs[:, :13], return_cache=True)
    sess = DecodeSession(m, cache, max_len=40)
    assert not sess.fused_gate
    for i in range(13, 40):
        with torch.no_grad():
            want, cache = m(xs[:, i:i + 1], cache=cache, return_cache=True)
        got = sess.step(xs[:, i:i + 1])
        assert_close(got, want, 2e-2, 1e-2, f"step {i}")
