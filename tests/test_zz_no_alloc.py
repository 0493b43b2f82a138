"""nsa_decode_attend_noalloc (split-K partials in the library's fixed device array, no allocation) against
nsa_decode_attend with a caller workspace, through the C ABI: the same kernels run with the same launch plan, so
the outputs and logits must be bit-equal.  Two calls in a row, the second on a smaller input, so that whatever the
first call left in the shared array would show; then the size limit."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _desc(q, k, v, mode, **kw):
    from native_sparse_attention_pytorch_amd import _lib
    b, hq, d = q.shape
    hk = k.shape[1]
    dsc = _lib.DecodeDesc()
    dsc.batch, dsc.kv_heads, dsc.group, dsc.dim_head = b, hk, hq // hk, d
    dsc.mode, dsc.scale = mode, d ** -0.5
    dsc.q_stride[:] = (q.stride(0), q.stride(1))
    dsc.k_stride[:] = k.stride()[:3]
    dsc.v_stride[:] = v.stride()[:3]
    for name, val in kw.items():
        setattr(dsc, name, val)
    return dsc


def _both(dsc, q, k, v, mem_k, mem_v, idx, fmask, want_logits):
    from native_sparse_attention_pytorch_amd import _lib
    L = _lib.lib()
    p = lambda t: 0 if t is None else t.data_ptr()
    st = torch.cuda.current_stream().cuda_stream
    nbytes = C.c_size_t()
    assert L.nsa_decode_workspace_bytes(C.byref(dsc), C.byref(nbytes)) == 0
    outs = []
    for noalloc in (False, True):
        out = torch.full(q.shape, float("nan"), dtype=torch.bfloat16, device=DEV)
        logits = torch.full((q.shape[0], q.shape[1], dsc.count), float("nan"), dtype=torch.float32, device=DEV) if want_logits else None
        if noalloc:
            rc = L.nsa_decode_attend_noalloc(C.byref(dsc), p(q), p(k), p(v), p(mem_k), p(mem_v), p(idx), p(fmask), p(out), p(logits), st)
        else:
            ws = torch.empty(max(nbytes.value, 16), dtype=torch.uint8, device=DEV)
            rc = L.nsa_decode_attend(C.byref(dsc), p(q), p(k), p(v), p(mem_k), p(mem_v), p(idx), p(fmask), p(ws), nbytes, p(out), p(logits), st)
        assert rc == 0, rc
        torch.cuda.synchronize()
        outs.append((out, logits))
    return outs, nbytes.value


def test_noalloc_decode_attend_matches_workspace_entry_point():
    from oracle import nsa_oracle as O
    g = torch.Generator().manual_seed(0)
    b, hq, hk, d, cap = 3, 8, 2, 128, 4100
    k = (torch.randn(b, hk, cap, d, generator=g) * d ** -0.25).to(torch.bfloat16).to(DEV)
    v = (torch.randn(b, hk, cap, d, generator=g) * d ** -0.25).to(torch.bfloat16).to(DEV)
    mem_k = torch.randn(hk, 2, d, generator=g).to(torch.bfloat16).to(DEV)
    mem_v = torch.randn(hk, 2, d, generator=g).to(torch.bfloat16).to(DEV)
    # first call: a long key range with memory rows and logits; second: a short one (fewer partial records)
    for count, start in ((4000, 37), (45, 3)):
        q = (torch.randn(b, hq, d, generator=g) * d ** -0.25).to(torch.bfloat16).to(DEV)
        dsc = _desc(q, k, v, 0, start=start, count=count, num_mem=2)
        print("noalloc range", count, flush=True)
        ((o1, l1), (o2, l2)), nbytes = _both(dsc, q, k, v, mem_k, mem_v, None, None, True)
        assert torch.isfinite(o2.float()).all() and torch.equal(o1, o2) and torch.equal(l1, l2), (count, nbytes)
        # and against the oracle's attention over the same keys (bf16 forward tolerance)
        kk = torch.cat((mem_k[None].expand(b, -1, -1, -1), k[:, :, start:start + count]), dim=2).float().cpu()
        vv = torch.cat((mem_v[None].expand(b, -1, -1, -1), v[:, :, start:start + count]), dim=2).float().cpu()
        want = O.attend(q.float().cpu()[:, :, None], kk, vv)[:, :, 0]
        assert (o2.float().cpu() - want).abs().max() < 2e-2
    # selected blocks + own block, then a smaller selection
    for S, kv_len in ((6, 4001), (2, 130)):
        q = (torch.randn(b, hq, d, generator=g) * d ** -0.25).to(torch.bfloat16).to(DEV)
        nblk = (kv_len - 1) // 64
        idx = torch.stack([torch.randperm(max(nblk, 1), generator=g)[:S] for _ in range(b * hk)]).reshape(b, hk, S).to(torch.int32).to(DEV)
        fmask = torch.ones(b, hk, S, dtype=torch.uint8, device=DEV)
        dsc = _desc(q, k, v, 1, block=64, num_sel=S, kv_len=kv_len)
        print("noalloc select", S, flush=True)
        ((o1, _), (o2, _)), _ = _both(dsc, q, k, v, None, None, idx, fmask, False)
        assert torch.isfinite(o2.float()).all() and torch.equal(o1, o2), (S, kv_len)


def test_noalloc_entry_point_leaves_device_memory_alone():
    """After a first call (which looks the array's address up), further calls neither take nor return device memory: the
    driver's free-memory figure and the caching allocator's counters are the same before and after."""
    from native_sparse_attention_pytorch_amd import _lib
    L = _lib.lib()
    g = torch.Generator().manual_seed(1)
    b, hq, hk, d, cap = 2, 8, 2, 128, 2100
    k = (torch.randn(b, hk, cap, d, generator=g) * d ** -0.25).to(torch.bfloat16).to(DEV)
    v = (torch.randn(b, hk, cap, d, generator=g) * d ** -0.25).to(torch.bfloat16).to(DEV)
    q = (torch.randn(b, hq, d, generator=g) * d ** -0.25).to(torch.bfloat16).to(DEV)
    out = torch.empty_like(q)
    dsc = _desc(q, k, v, 0, start=0, count=2000, num_mem=0)
    st = torch.cuda.current_stream().cuda_stream
    call = lambda: L.nsa_decode_attend_noalloc(C.byref(dsc), q.data_ptr(), k.data_ptr(), v.data_ptr(), 0, 0, 0, 0, out.data_ptr(), 0, st)
    assert call() == 0
    torch.cuda.synchronize()
    first = out.clone()
    before = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    for _ in range(3):
        assert call() == 0
    torch.cuda.synchronize()
    after = (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved())
    assert before == after, (before, after)
    assert torch.equal(out, first)


def test_noalloc_rejects_sizes_beyond_its_array():
    from native_sparse_attention_pytorch_amd import _lib
    L = _lib.lib()
    b, hq, hk, d, cap = 64, 32, 8, 128, 64
    q = torch.zeros(b, hq, d, dtype=torch.bfloat16, device=DEV)
    k = torch.zeros(b, hk, cap, d, dtype=torch.bfloat16, device=DEV)
    dsc = _desc(q, k, k, 0, start=0, count=32768, num_mem=0)       # never launched: the size check comes first
    nbytes = C.c_size_t()
    assert L.nsa_decode_workspace_bytes(C.byref(dsc), C.byref(nbytes)) == 0
    assert nbytes.value > (16 << 20)
    out = torch.zeros_like(q)
    rc = L.nsa_decode_attend_noalloc(C.byref(dsc), q.data_ptr(), k.data_ptr(), k.data_ptr(), 0, 0, 0, 0, out.data_ptr(), 0,
                                     torch.cuda.current_stream().cuda_stream)
    assert rc == -3
