"""Host logic of the growing decode caches (no GPU): a cache tensor is the filled prefix of a
buffer with spare rows; appending takes a spare row in place, and any tensor that is not the
live prefix of such a buffer (a prefill cache, an older tuple at a branch point, a full buffer)
is copied into a new buffer first, so tensors handed out earlier never change."""
import torch

from native_sparse_attention_pytorch_amd.sparse_attention import _append_rows


def test_first_append_copies_then_appends_in_place():
    t = torch.randn(2, 3, 5, 8).to(torch.bfloat16)              # e.g. the cache the parallel forward returned
    grown, row = _append_rows(t)
    assert grown.shape == (2, 3, 6, 8) and row.shape == (2, 3, 1, 8)
    assert torch.equal(grown[:, :, :5], t) and grown._base is not None and grown._base.shape[2] >= 12
    row.fill_(1.0)
    base = grown._base
    grown2, row2 = _append_rows(grown)
    assert grown2._base is base, "second append must reuse the buffer"
    assert grown2.data_ptr() == grown.data_ptr() and torch.equal(grown2[:, :, :6], grown)
    assert row2.data_ptr() == base[:, :, 6:7].data_ptr()


def test_branching_from_an_older_cache_copies():
    t = torch.zeros(1, 1, 4, 8, dtype=torch.bfloat16)
    a, ra = _append_rows(t)
    ra.fill_(1.0)
    b, rb = _append_rows(a)          # advances the shared buffer to 6 rows
    rb.fill_(2.0)
    c, rc = _append_rows(a)          # `a` is no longer the live prefix: must not overwrite b's row
    rc.fill_(3.0)
    assert c._base is not b._base
    assert float(b[0, 0, 5, 0]) == 2.0 and float(c[0, 0, 5, 0]) == 3.0
    assert torch.equal(c[:, :, :5], a) and torch.equal(b[:, :, :5], a)


def test_growth_when_capacity_is_exhausted_and_dtype_policy():
    t = torch.randn(1, 2, 3, 8)                                   # fp32 cache from an fp32 module: converted once
    cur, _ = _append_rows(t, min_capacity=4)
    assert cur.dtype == torch.bfloat16
    bases = {id(cur._base)}
    for _ in range(40):
        cur, row = _append_rows(cur, min_capacity=4)
        row.zero_()
        bases.add(id(cur._base))
    assert cur.shape[2] == 44
    assert 2 <= len(bases) <= 6, "doubling growth: a handful of reallocations for 40 appends"
    keep, _ = _append_rows(torch.randn(1, 2, 3, 8), dtype=torch.float32, min_capacity=16)
    assert keep.dtype == torch.float32 and keep._base.shape[2] == 16


def test_empty_cache_and_views_that_do_not_start_at_the_buffer():
    e = torch.zeros(2, 2, 0, 8, dtype=torch.bfloat16)
    g, row = _append_rows(e)
    assert g.shape[2] == 1
    g2, _ = _append_rows(g)
    tail = g2[:, :, 1:]              # a suffix view (what the running window keeps after a compression step)
    h, _ = _append_rows(tail)
    assert h._base is not g2._base and h.shape[2] == 2


def test_ring_rows_hold_the_last_positions():
    """The graph-replayed decode keeps the un-rotated keys of the last tokens in a ring (position p in row p % ring);
    the compression window ending at position `end` must read exactly positions end-cbs .. end-1, zeros before the
    sequence start, for every alignment and across the wrap."""
    from native_sparse_attention_pytorch_amd.decode_session import ring_rows
    for cbs, st in ((8, 4), (16, 16), (32, 8), (5, 5)):
        ring = 2 * cbs
        buf = torch.zeros(ring)
        ar = torch.arange(cbs, dtype=torch.int32)
        for pos in range(5 * ring + 3):
            buf[pos % ring] = pos + 1                         # value = position + 1, so that 0 means "never written"
            end = pos + 1
            if end % st:
                continue
            for first in (end - cbs, torch.tensor(end - cbs, dtype=torch.int32)):      # host int and device-style counter
                rows = ring_rows(first, ar, ring)
                got = buf[rows.long()]
                want = torch.tensor([float(p + 1) if p >= 0 else 0.0 for p in range(end - cbs, end)])
                assert torch.equal(got, want), (cbs, st, pos)


def test_group_padding_round_trip():
    """Query heads of a kv group are padded to a power of two with zero heads at the end of each group, and come back
    in their original order."""
    from native_sparse_attention_pytorch_amd.ops import _pad_groups, _unpad_groups
    for hk, g in ((2, 3), (1, 5), (4, 6), (3, 7), (2, 4), (5, 1)):
        q = torch.randn(2, hk * g, 7, 8)
        qp, g0, gp = _pad_groups(q, hk)
        assert g0 == g and gp >= g and gp & (gp - 1) == 0 and gp < 2 * g + (g == 1)
        assert qp.shape == (2, hk * gp, 7, 8)
        grouped = qp.reshape(2, hk, gp, 7, 8)
        assert torch.equal(grouped[:, :, :g].reshape(2, hk * g, 7, 8), q)
        assert (grouped[:, :, g:] == 0).all()
        assert torch.equal(_unpad_groups(qp, hk, g, gp), q)
        lse = torch.randn(2, hk * gp, 7)
        assert _unpad_groups(lse, hk, g, gp).shape == (2, hk * g, 7)


def test_append_rows_into_wider_buffers():
    """A cache of d features moves into a buffer of `feat` >= d features (the padding stays zero) and grows in place
    from then on."""
    from native_sparse_attention_pytorch_amd.sparse_attention import _append_rows
    t = torch.randn(2, 3, 5, 40).to(torch.bfloat16)
    full, row = _append_rows(t, feat=64)
    assert full.shape == (2, 3, 6, 64) and row.shape == (2, 3, 1, 64)
    assert torch.equal(full[:, :, :5, :40], t) and (full[:, :, :5, 40:] == 0).all()
    row.copy_(torch.ones_like(row))
    again, row2 = _append_rows(full, feat=64)
    assert again.data_ptr() == full.data_ptr() and again.shape == (2, 3, 7, 64)       # in place: same buffer
    assert torch.equal(again[:, :, 5], torch.ones(2, 3, 64, dtype=torch.bfloat16))
