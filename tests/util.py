"""Shared helpers for the parity tests."""
import contextlib
import math

import torch


def causal_random_selection(b, h, n, B, S, seed, own_reserved=0):
    """For query i in block w = i // B: min(w, S) distinct blocks drawn uniformly from [0, w)
    (random-score top-k), remaining slots dead.  Vectorised; CPU int64/bool tensors."""
    g = torch.Generator().manual_seed(seed)
    W = math.ceil(n / B)
    scores = torch.rand(b, h, n, W, generator=g)
    blk = (torch.arange(n) // B)[None, None, :, None]
    scores = scores.masked_fill(torch.arange(W)[None, None, None, :] >= blk, -1.0)
    k = min(S, W)
    vals, idx = scores.topk(k, dim=-1)
    mask = vals >= 0
    if k < S:
        idx = torch.nn.functional.pad(idx, (0, S - k))
        mask = torch.nn.functional.pad(mask, (0, S - k))
    idx = idx.masked_fill(~mask, 0)
    return idx, mask


def rel_err(a, b):
    return ((a.float() - b.float()).abs().max() / b.float().abs().max().clamp_min(1e-12)).item()


def assert_close(got, want, atol, rtol, what=""):
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs()
    tol = atol + rtol * want.abs()
    bad = err > tol
    if bad.any():
        i = torch.nonzero(bad)[0].tolist()
        raise AssertionError(f"{what}: {int(bad.sum())}/{bad.numel()} elements out of tolerance; "
                             f"max err {err.max().item():.4g} (ref max {want.abs().max().item():.4g}); first at {i}: "
                             f"got {got[tuple(i)].item():.6g} want {want[tuple(i)].item():.6g}")


def assert_grad_close(got, want, what="", elem_floor=1e-2):
    """Gradient bound used by the kernel tests: 5e-2 relative in the norm of the whole tensor (the stated bound), and per
    element 5e-2 relative with an absolute floor of 1e-2 of the tensor's largest entry (a relative bound alone is
    meaningless for the entries near zero)."""
    g, w = got.float().cpu(), want.float().cpu()
    # a gradient that is zero in exact arithmetic (one visible key: softmax = 1) comes out as rounding noise; 1e-6 per
    # element is the absolute floor below which the relative figure means nothing
    err, floor = (g - w).norm().item(), 1e-6 * w.numel() ** 0.5
    e = err / max(w.norm().item(), 1e-12)
    assert e < 5e-2 or err <= floor, f"{what}: relative error {e:.4f} (norm-wise) exceeds 5e-2"
    assert_close(got, want, elem_floor * w.abs().max().item() + 1e-6, 5e-2, what)


@contextlib.contextmanager
def capture_selection(captured):
    """While active, the block selection the module makes - through `ops.importance_topk` (logits written out) or
    `ops.compress_attend_topk` (selection inside the compressed forward) - is recorded in captured["sel"] as CPU
    (idx int64, fmask bool), and captured["via"] names the path."""
    from native_sparse_attention_pytorch_amd import ops
    orig_topk, orig_fused = ops.importance_topk, ops.compress_attend_topk

    def spy_topk(imp, k, **kw):
        r = orig_topk(imp, k, **kw)
        captured["sel"], captured["via"] = (r[1].cpu().long(), r[2].cpu()), "importance_topk"
        return r

    def spy_fused(*a, **kw):
        r = orig_fused(*a, **kw)
        captured["sel"], captured["via"] = (r[1].cpu().long(), r[2].cpu()), "compress_attend_topk"
        return r
    ops.importance_topk, ops.compress_attend_topk = spy_topk, spy_fused
    try:
        yield captured
    finally:
        ops.importance_topk, ops.compress_attend_topk = orig_topk, orig_fused
