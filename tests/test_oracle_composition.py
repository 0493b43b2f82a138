"""Pins for the two composite functions of the oracle, written without any of the oracle's own
building blocks, so that a mistake in how the blocks are wired (which branch sees rotated q / k,
which input feeds the gate, where the memory slots go, a dropped residual, a wrong label shift)
fails here.

  SparseAttentionOracle.forward   <- native_sparse_attention.py:549-867, rebuilt below from
      F.scaled_dot_product_attention under the three dense masks of native_sparse_attention.py:46-109,
      rotary as a complex multiplication, windows and importance scores by python loops.
  TransformerOracle.forward       <- transformer.py:130-138, 254-330, rebuilt from its closed forms:
      depth 0, residual structure with silenced sub-layers, one hand-rolled layer, hand-written
      cross entropy with the [:, :-1] / [:, 1:] shift.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import nsa_oracle as O


# ----------------------------------------------------------------- independent building blocks

def rms_norm(x, w):
    # nn.RMSNorm(dim) with eps=None: eps = finfo(dtype).eps
    return x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + torch.finfo(x.dtype).eps) * w


def heads_of(t, d):
    # 'b n (h d) -> b h n d'
    b, n, hd = t.shape
    return torch.stack([t[:, :, h * d:(h + 1) * d] for h in range(hd // d)], dim=1)


def rope_complex(t, theta=10000.0, offset=0):
    """Feature pair (2k, 2k+1) as the complex number x + iy, multiplied by exp(i * pos * theta^(-2k/d))."""
    d, n = t.shape[-1], t.shape[-2]
    z = torch.view_as_complex(t.double().reshape(*t.shape[:-1], d // 2, 2).contiguous())
    freqs = theta ** (-torch.arange(0, d, 2, dtype=torch.float64) / d)
    ang = (torch.arange(n, dtype=torch.float64) + offset)[:, None] * freqs[None, :]
    out = z * torch.polar(torch.ones_like(ang), ang)
    return torch.view_as_real(out).reshape(t.shape).to(t.dtype)


def sdpa_gqa(q, k, v, mask, g):
    """Library attention; kv head h serves query heads h*g .. h*g+g-1 (NSA.py:164, 848)."""
    k, v = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    return F.scaled_dot_product_attention(q, k, v, attn_mask=mask)


def module_forward_from_scratch(m, x):
    """SparseAttention.forward (NSA.py:549-867, torch path) for a module with the default networks,
    read off the reference line by line; returns the output and the selected blocks."""
    b, n, _ = x.shape
    d, Hq, Hkv, G = m.dim_head, m.heads, m.kv_heads, m.num_grouped_queries
    st, cbs, B, S, M = (m.compress_block_sliding_stride, m.compress_block_size, m.selection_block_size,
                        m.num_selected_blocks, m.num_mem_compress_kv)
    causal, scale = m.causal, d ** -0.5
    sd = {k_: v_.detach() for k_, v_ in m.state_dict().items()}

    xin = rms_norm(x, sd["norm.weight"])                                            # :579
    qkv = xin @ sd["to_qkv.weight"].T                                               # :583
    q = heads_of(qkv[..., :Hq * d], d)
    k = heads_of(qkv[..., Hq * d:(Hq + Hkv) * d], d)
    v = heads_of(qkv[..., (Hq + Hkv) * d:], d)                                      # :585

    # compressed keys / values from the UN-ROTATED k, v (:589-614); window w = tokens (w+1)st-cbs .. (w+1)st-1
    nc = n // st
    def compress(t, pos, prefix):
        out = torch.zeros(b, Hkv, nc, d)
        for w in range(nc):
            win = torch.zeros(b, Hkv, cbs, d)
            for r in range(cbs):
                tok = (w + 1) * st - cbs + r
                if tok >= 0:
                    win[:, :, r] = t[:, :, tok]
            win = win + pos[None]                                                   # :600-601
            h1 = torch.relu(win.reshape(b, Hkv, cbs * d) @ sd[prefix + ".1.weight"].T + sd[prefix + ".1.bias"])
            out[:, :, w] = h1 @ sd[prefix + ".3.weight"].T + sd[prefix + ".3.bias"]
        return out
    ck = compress(k, sd["k_intrablock_positions"], "k_compress")
    cv = compress(v, sd["v_intrablock_positions"], "v_compress")
    ck = torch.cat((sd["compress_mem_kv"][0][None].expand(b, -1, -1, -1), ck), dim=2)   # :621-626 memory slots first
    cv = torch.cat((sd["compress_mem_kv"][1][None].expand(b, -1, -1, -1), cv), dim=2)

    # 1. compressed attention, un-rotated q (:632-639)
    cmask = torch.ones(n, M + nc, dtype=torch.bool)
    if causal:
        for i in range(n):
            for c in range(nc):
                cmask[i, M + c] = (c + 1) * st - 1 < i
    c_out = sdpa_gqa(q, ck, cv, cmask, G)

    # importance scores from the same logits (:652-695)
    sim = torch.einsum("bhid,bhjd->bhij", q, ck.repeat_interleave(G, dim=1)) * scale
    sim = sim.masked_fill(~cmask, -torch.finfo(sim.dtype).max // 10)                # :171
    imp = sim[..., M:]
    if m.query_heads_share_selected_kv:
        imp = torch.stack([imp[:, h * G:(h + 1) * G].mean(dim=1) for h in range(Hkv)], dim=1)   # :660
    num_sel = min(S, nc)
    if st != B:
        npf = B // st
        nb = nc // npf
        pooled = torch.zeros(*imp.shape[:-1], nb)
        for j in range(nb):
            pooled[..., j] = imp[..., j * npf:(j + 1) * npf].mean(dim=-1)           # :676-680
        for i in range(n):
            if i // B < nb:
                pooled[:, :, i, i // B] = -torch.finfo(sim.dtype).max               # :686-691
        imp = pooled
    probs = F.pad(imp, (1, 0), value=-1e3).softmax(dim=-1)[..., 1:]                 # :693-695
    num_sel = min(num_sel, probs.shape[-1])

    # rotary for branches 2 and 3 only (:643)
    rq, rk = rope_complex(q), rope_complex(k)

    # 2. selected blocks (:741-819) as the dense mask of :90-104
    W = math.ceil(n / B)
    Hs = probs.shape[1]
    blk_of = torch.arange(n) // B
    if num_sel > 0:
        vals, idx = probs.topk(num_sel, dim=-1)                                     # :713
        live = vals > 1e-10                                                         # :721 / :742
        chosen = torch.zeros(b, Hs, n, W, dtype=torch.bool)
        for s in range(num_sel):
            chosen.scatter_(-1, idx[..., s:s + 1], live[..., s:s + 1] | chosen.gather(-1, idx[..., s:s + 1]))
        sel = chosen[..., blk_of]                                                   # key j -> its block
        if causal:
            i_, j_ = torch.arange(n)[:, None], torch.arange(n)[None, :]
            fmask = (i_ >= j_) & ((blk_of[:, None] == blk_of[None, :]) | sel)
        else:
            fmask = sel
    else:
        idx = live = None
        fmask = blk_of[:, None] == blk_of[None, :]                                  # :821-837
        if causal:
            fmask = fmask & (torch.arange(n)[:, None] >= torch.arange(n)[None, :])
        fmask = fmask[None, None].expand(b, Hs, n, n)
    if Hs == Hkv:
        fmask = fmask.repeat_interleave(G, dim=1)
    f_out = sdpa_gqa(rq, rk, v, fmask, G)

    # 3. sliding window (:841-850) as the mask of :48-56
    dist = torch.arange(n)[:, None] - torch.arange(n)[None, :]
    smask = (dist <= m.sliding_window_size) & (dist >= (0 if causal else -m.sliding_window_size))
    s_out = sdpa_gqa(rq, rk, v, smask, G)

    # gate from the NORMED input (:854-856), column h*3+s, s = compressed, fine, sliding
    gl = torch.sigmoid(xin @ sd["to_strategy_combine.0.weight"].T + sd["to_strategy_combine.0.bias"])
    out = torch.zeros(b, n, Hq * d)
    for h in range(Hq):
        out[:, :, h * d:(h + 1) * d] = (gl[:, :, 3 * h:3 * h + 1] * c_out[:, h] + gl[:, :, 3 * h + 1:3 * h + 2] * f_out[:, h]
                                        + gl[:, :, 3 * h + 2:3 * h + 3] * s_out[:, h])       # :856, :860
    return out @ sd["combine_heads.weight"].T, idx, live                            # :862


def _randomised(m, seed):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():                  # every parameter away from its symmetric / zero init
        m.to_strategy_combine[0].weight.copy_(torch.randn(m.to_strategy_combine[0].weight.shape, generator=g) * 0.3)
        m.to_strategy_combine[0].bias.copy_(torch.randn(m.to_strategy_combine[0].bias.shape, generator=g))
        m.compress_mem_kv.copy_(torch.randn(m.compress_mem_kv.shape, generator=g))
        m.k_intrablock_positions.copy_(torch.randn(m.k_intrablock_positions.shape, generator=g))
        m.v_intrablock_positions.copy_(torch.randn(m.v_intrablock_positions.shape, generator=g))
        m.norm.weight.copy_(1.0 + 0.3 * torch.randn(m.norm.weight.shape, generator=g))
        for p in m.v_compress.parameters():
            p.add_(torch.randn(p.shape, generator=g) * 0.05)
    return m


COMPOSE = [
    # causal, n, heads, kv_heads, B, cbs, st, S, share, window
    (True, 29, 4, 2, 4, 4, 2, 2, True, 3),
    (False, 24, 4, 2, 4, 4, 2, 2, True, 3),
    (True, 33, 4, 4, 8, 8, 8, 2, True, 5),          # stride == block: no pooling, no own-block fill
    (True, 26, 4, 2, 8, 4, 2, 3, False, 2),         # per-head selection
    (False, 20, 2, 1, 4, 6, 2, 1, True, 1),
    (True, 21, 4, 2, 4, 4, 2, 0, True, 3),          # nothing selected: block-diagonal fallback
    (True, 3, 2, 2, 4, 4, 2, 2, True, 2),           # shorter than one block
]


@pytest.mark.parametrize("causal,n,heads,kvh,B,cbs,st,S,share,win", COMPOSE)
def test_module_forward_equals_rebuild_from_library_attention(causal, n, heads, kvh, B, cbs, st, S, share, win):
    torch.manual_seed(n + B)
    m = O.SparseAttentionOracle(dim=32, dim_head=8, heads=heads, kv_heads=kvh, sliding_window_size=win, compress_block_size=cbs,
                                compress_block_sliding_stride=st, selection_block_size=B, num_selected_blocks=S, causal=causal,
                                query_heads_share_selected_kv=share, num_compressed_mem_kv=2)
    _randomised(m, n)
    x = torch.randn(2, n, 32)
    got, parts = m(x, return_parts=True)
    want, idx, live = module_forward_from_scratch(m, x)
    assert torch.allclose(got, want, atol=2e-5, rtol=1e-4), (got - want).abs().max()
    if idx is not None and parts["idx"] is not None:
        olive = parts["vals"] > 1e-10
        for a, la, o, lo in zip(idx.flatten(0, 2), live.flatten(0, 2), parts["idx"].flatten(0, 2), olive.flatten(0, 2)):
            assert set(a[la].tolist()) == set(o[lo].tolist())


def test_rebuild_detects_miswiring():
    """The rebuild is sensitive to the wiring it is meant to pin: feeding rotated queries to the compressed
    branch, or the un-normed input to the gate, moves the output by far more than the tolerance above."""
    torch.manual_seed(1)
    m = _randomised(O.SparseAttentionOracle(dim=32, dim_head=8, heads=4, kv_heads=2, sliding_window_size=3, compress_block_size=4,
                                            compress_block_sliding_stride=2, selection_block_size=4, num_selected_blocks=2, causal=True), 7)
    x = torch.randn(1, 29, 32)
    base = m(x)
    x_in, q, k, v = m.project(x)
    ck, cv = m.compress(k, v)
    rq = rope_complex(q)
    cm = O.compress_mask(29, ck.shape[-2] - 1, 2, 1, True)
    delta_c = (O.attend(rq, ck, cv, mask=cm) - O.attend(q, ck, cv, mask=cm)).abs().max()
    assert delta_c > 1e-3
    g_raw = m.to_strategy_combine(x)
    g_norm = m.to_strategy_combine(x_in)
    assert (g_raw - g_norm).abs().max() > 1e-3
    assert torch.isfinite(base).all()


# --------------------------------------------------------------------------- transformer harness

def _tiny_transformer(depth, seed=0):
    torch.manual_seed(seed)
    return O.TransformerOracle(num_tokens=17, dim=32, depth=depth, dim_head=8, heads=4, kv_heads=2, causal=True,
                               sparse_attn_kwargs=dict(sliding_window_size=3, compress_block_size=4, compress_block_sliding_stride=2,
                                                       selection_block_size=4, num_selected_blocks=2))


def hand_cross_entropy(logits, labels):
    # mean over every (batch, position) of -log softmax(logits)[label]
    total = 0.0
    b, n, _ = logits.shape
    for bi in range(b):
        for t in range(n):
            row = logits[bi, t].double()
            total += (torch.logsumexp(row, dim=0) - row[labels[bi, t]]).item()
    return total / (b * n)


def test_transformer_depth0_closed_form():
    """transformer.py:264-330 with no layers: loss = CE(to_logits(RMSNorm(emb(ids[:, :-1]))), ids[:, 1:])."""
    model = _tiny_transformer(0)
    with torch.no_grad():
        model.norm.weight.copy_(1.0 + 0.2 * torch.randn(32))
    ids = torch.randint(0, 17, (3, 12))
    loss = model(ids, return_loss=True).item()
    emb = model.token_emb.weight.detach()[ids[:, :-1]]
    logits = rms_norm(emb, model.norm.weight.detach()) @ model.to_logits.weight.detach().T
    assert abs(loss - hand_cross_entropy(logits, ids[:, 1:])) < 1e-5
    # the shift matters: scoring position t against token t (no shift) or t+2 gives another number
    assert abs(loss - hand_cross_entropy(logits, ids[:, :-1])) > 1e-3
    # without return_loss the whole sequence is embedded and logits come back
    full = model(ids)
    assert full.shape == (3, 12, 17)
    assert torch.allclose(full[:, :-1], logits, atol=1e-5)


def test_transformer_residual_structure():
    """transformer.py:317-318: tokens = attn(tokens) + tokens; tokens = ff(tokens) + tokens.  With the attention's
    output projection and the feed-forward's last layer silenced both sub-layers add zero: the loss equals depth 0.
    Silencing only one of the two leaves exactly the other's residual update."""
    model = _tiny_transformer(2, seed=3)
    ids = torch.randint(0, 17, (2, 14))
    emb = model.token_emb.weight.detach()[ids[:, :-1]]
    final = lambda t: rms_norm(t, model.norm.weight.detach()) @ model.to_logits.weight.detach().T
    with torch.no_grad():
        for attn, ff in model.layers:
            attn.combine_heads.weight.zero_()
            ff[3].weight.zero_()
            ff[3].bias.zero_()
    assert abs(model(ids, return_loss=True).item() - hand_cross_entropy(final(emb), ids[:, 1:])) < 1e-5
    # feed-forward of layer 0 alive: tokens = emb + W2 gelu(W1 rmsnorm(emb) + b1) + b2 (transformer.py:130-138)
    with torch.no_grad():
        ff = model.layers[0][1]
        ff[3].weight.copy_(torch.randn(32, 128) * 0.2)
        ff[3].bias.copy_(torch.randn(32) * 0.1)
    h = rms_norm(emb, ff[0].weight.detach()) @ ff[1].weight.detach().T + ff[1].bias.detach()
    gelu = 0.5 * h * (1.0 + torch.erf(h / math.sqrt(2.0)))
    tok = emb + gelu @ ff[3].weight.detach().T + ff[3].bias.detach()
    assert abs(model(ids, return_loss=True).item() - hand_cross_entropy(final(tok), ids[:, 1:])) < 1e-5


def test_transformer_one_layer_hand_rolled():
    """One full layer: the attention sub-layer's output is the (separately pinned) sparse attention of the raw token
    embeddings - pre-norm happens inside it - added to them, then the feed-forward residual, final norm, logits."""
    model = _tiny_transformer(1, seed=5)
    with torch.no_grad():
        _randomised(model.layers[0][0], 11)
    ids = torch.randint(0, 17, (2, 19))
    emb = model.token_emb.weight.detach()[ids[:, :-1]]
    attn, ff = model.layers[0]
    a_out, _, _ = module_forward_from_scratch(attn, emb)
    tok = emb + a_out
    h = rms_norm(tok, ff[0].weight.detach()) @ ff[1].weight.detach().T + ff[1].bias.detach()
    tok = tok + (0.5 * h * (1.0 + torch.erf(h / math.sqrt(2.0)))) @ ff[3].weight.detach().T + ff[3].bias.detach()
    logits = rms_norm(tok, model.norm.weight.detach()) @ model.to_logits.weight.detach().T
    assert abs(model(ids, return_loss=True).item() - hand_cross_entropy(logits, ids[:, 1:])) < 2e-5
    # the cached path embeds only the last token and must give the same last-position logits
    lg, cache = model(ids[:, :10], return_cache=True)
    lg2, _ = model(ids[:, :11], cache=cache, return_cache=True)
    full = model(ids[:, :11])
    assert torch.allclose(lg2[:, -1], full[:, -1], atol=1e-5)


# ------------------------------------------------------------------------- dtype-faithful mode

def test_oracle_in_bf16_is_the_same_function_at_bf16_precision():
    """The oracle cast to bf16 (fill values, pad, softmaxes and GEMMs in that dtype, as the reference's torch path runs
    when its module is cast) stays within the bf16 forward bound of the fp32 oracle under the same block selection, and
    its masks hold exactly: a fully masked key gets probability 0 in bf16 as well (causality is not a matter of precision)."""
    import copy
    torch.manual_seed(4)
    m = _randomised(O.SparseAttentionOracle(dim=64, dim_head=16, heads=4, kv_heads=2, sliding_window_size=6, compress_block_size=8,
                                            compress_block_sliding_stride=4, selection_block_size=8, num_selected_blocks=2, causal=True), 3)
    with torch.no_grad():
        for p in m.parameters():
            p.copy_(p.bfloat16().float())
    x = torch.randn(2, 70, 64).bfloat16()
    y32, parts = m(x.float(), return_parts=True)
    sel = (parts["idx"], parts["vals"] > 1e-10)
    m16 = copy.deepcopy(m).to(torch.bfloat16)
    y16 = m16(x, selection_override=sel)
    assert y16.dtype == torch.bfloat16
    assert ((y16.float() - y32).abs() <= 2e-2 + 1e-2 * y32.abs()).all()
    x2 = x.clone()
    x2[:, 40:] += 1.0
    y16b = m16(x2, selection_override=sel)
    assert torch.equal(y16[:, :40], y16b[:, :40])
