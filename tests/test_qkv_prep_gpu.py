"""The fused epilogue of the qkv projection (head split + rotation of q / k + compression windows with
positions + casts, one kernel each way) against the oracle's restatements of those steps
(NSA.py:583-614, 643), forward and backward, for bf16 and fp32 projections."""
import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import assert_close, assert_grad_close

pytestmark = pytest.mark.gpu
DEV = "cuda"

CASES = [
    # b, n, hq, hk, d, cbs, st, offset, dtype
    (2, 100, 4, 2, 64, 16, 8, 0, torch.bfloat16),
    (1, 333, 8, 2, 128, 32, 16, 0, torch.bfloat16),
    (2, 64, 3, 3, 64, 8, 8, 0, torch.float32),
    (1, 50, 4, 1, 64, 24, 4, 7, torch.float32),
    (1, 5, 2, 2, 128, 8, 8, 0, torch.bfloat16),          # fewer tokens than one window step: no windows
    (1, 515, 4, 2, 128, 16, 4, 40000, torch.float32),    # large positions: sine / cosine range reduction
]


@pytest.mark.parametrize("b,n,hq,hk,d,cbs,st,offset,dtype", CASES)
def test_qkv_prep_matches_oracle(b, n, hq, hk, d, cbs, st, offset, dtype):
    from native_sparse_attention_pytorch_amd.ops import qkv_prep
    g = torch.Generator().manual_seed(n * 7 + d + cbs)
    width = (hq + 2 * hk) * d
    qkv = torch.randn(b, n, width, generator=g).to(dtype)
    kpos, vpos = (torch.randn(hk, cbs, d, generator=g) * 0.3).to(dtype), (torch.randn(hk, cbs, d, generator=g) * 0.3).to(dtype)
    rot = O.RotaryEmbedding(d)

    # oracle side, fp32 (NSA.py:583-603, 643)
    ref_in = qkv.float().clone().requires_grad_()
    kp_r, vp_r = kpos.float().clone().requires_grad_(), vpos.float().clone().requires_grad_()
    q, k, v = ref_in.split((hq * d, hk * d, hk * d), dim=-1)
    q, k, v = (O.split_heads(t, d) for t in (q, k, v))
    L = (n // st) * st
    kw_r, vw_r = O.compress_windows(k[..., :L, :], cbs, st), O.compress_windows(v[..., :L, :], cbs, st)
    if kw_r.numel():
        kw_r, vw_r = kw_r + kp_r[None, :, None], vw_r + vp_r[None, :, None]
    rq_r, rk_r = rot.rotate(q, offset=offset), rot.rotate(k, offset=offset)
    want = (q, rq_r, rk_r, v, kw_r, vw_r)

    dev_in = qkv.to(DEV).requires_grad_()
    kp_g, vp_g = kpos.to(DEV).requires_grad_(), vpos.to(DEV).requires_grad_()
    got = qkv_prep(dev_in, rot.freqs.to(DEV), kp_g, vp_g, hq, hk, d, cbs, st, offset)
    torch.cuda.synchronize()
    names = ("q", "rotated q", "rotated k", "v", "k windows", "v windows")
    for nm, a, r in zip(names, got, want):
        assert a.shape == r.shape, nm
        if r.numel() == 0:
            continue
        assert a.dtype == (dtype if "windows" in nm else torch.bfloat16), nm
        tol = 1e-5 if (dtype == torch.float32 and "windows" in nm) else 1.6e-2 * r.abs().max().item()
        assert_close(a, r.detach(), tol, 1e-2 if tol > 1e-4 else 1e-5, nm)

    # backward: independent upstream gradients into all six outputs
    gs = [torch.randn(r.shape, generator=g) for r in want]
    gs_dev = [x.to(DEV).to(a.dtype) for x, a in zip(gs, got)]
    loss_r = sum((r * x.to(torch.bfloat16 if a.dtype == torch.bfloat16 else torch.float32).float()).sum() for r, x, a in zip(want, gs, got))
    loss_r.backward()
    sum((a.float() * x.float()).sum() for a, x in zip(got, gs_dev)).backward()
    torch.cuda.synchronize()
    assert dev_in.grad.dtype == dtype and dev_in.grad.shape == qkv.shape
    assert_grad_close(dev_in.grad, ref_in.grad, "d qkv")
    if kw_r.numel():
        assert_grad_close(kp_g.grad, kp_r.grad, "d k positions")
        assert_grad_close(vp_g.grad, vp_r.grad, "d v positions")


def test_qkv_prep_partial_gradients():
    """Outputs that take no part in the loss contribute zero (their gradients reach the kernel as NULL)."""
    from native_sparse_attention_pytorch_amd.ops import qkv_prep
    g = torch.Generator().manual_seed(3)
    b, n, hq, hk, d, cbs, st = 1, 40, 2, 1, 64, 8, 4
    qkv = torch.randn(b, n, (hq + 2 * hk) * d, generator=g).bfloat16().to(DEV).requires_grad_()
    kpos = torch.zeros(hk, cbs, d, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    rot = O.RotaryEmbedding(d)
    outs = qkv_prep(qkv, rot.freqs.to(DEV), kpos, kpos, hq, hk, d, cbs, st)
    outs[3].float().sum().backward()                     # only v
    torch.cuda.synchronize()
    gq = qkv.grad.float()
    assert (gq[..., :(hq + hk) * d] == 0).all() and (gq[..., (hq + hk) * d:] == 1).all()
    assert kpos.grad is None or (kpos.grad == 0).all()
