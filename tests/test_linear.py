"""ops.linear: the projections' weight gradient as a GEMM over slices of the token axis.  It computes what autograd's own
F.linear backward computes (NSA.py:583, 853, 858 are plain nn.Linear calls), so the checks are against torch itself."""
import pytest
import torch
import torch.nn.functional as F

from native_sparse_attention_pytorch_amd import ops


def test_slices_by_shape():
    assert ops._wgrad_splits(16384, 1024, 1024) == 8
    assert ops._wgrad_splits(16384, 1024, 1536) == 8
    assert ops._wgrad_splits(16384, 1024, 48) == 8
    assert ops._wgrad_splits(4080, 2048, 2048) == 1        # 256 tiles already
    assert ops._wgrad_splits(4080, 2048, 64) == 1          # too few tokens a slice
    assert ops._wgrad_splits(4096, 1024, 1024) == 1        # a short token axis: the GEMM is microseconds, a second launch is not worth it
    assert ops._wgrad_splits(32768, 1024, 1024) == 8
    assert ops._wgrad_splits(8192, 512, 512) == 8          # a config-5 step: 8 x 1024 tokens
    assert ops._wgrad_splits(8192, 512, 2048) == 8
    assert ops._wgrad_splits(4096, 1024, 64, replayed=True) == 4      # recorded into a graph: launches are free at replay
    assert ops._wgrad_splits(16384, 512, 512, replayed=True) == 16
    assert ops._wgrad_splits(2048, 1024, 64, replayed=True) == 1
    assert ops._wgrad_splits(16383, 1024, 1024) == 1       # no even cut
    assert ops._wgrad_splits(2048, 64, 64) == 1


def test_whole_gemm_path_equals_autograd_cpu():
    torch.manual_seed(0)
    x = torch.randn(3, 37, 24, requires_grad=True)
    w = torch.randn(40, 24, requires_grad=True)
    b = torch.randn(40, requires_grad=True)
    dy = torch.randn(3, 37, 40)
    ref = torch.autograd.grad(F.linear(x, w, b), (x, w, b), dy)
    got = torch.autograd.grad(ops.linear(x, w, b), (x, w, b), dy)
    for r, g in zip(ref, got):
        torch.testing.assert_close(g, r, rtol=1e-5, atol=1e-5)
    assert torch.equal(ops.linear(x, w, b), F.linear(x, w, b))
    with torch.no_grad():
        assert torch.equal(ops.linear(x, w), F.linear(x, w))


@pytest.mark.gpu
@pytest.mark.parametrize("rows,n_in,n_out,bias", [(16384, 1024, 1536, False), (32768, 512, 48, True), (16384, 256, 1024, False),
                                                  ((8, 2048), 128, 320, True)])
def test_sliced_weight_gradient_equals_autograd(rows, n_in, n_out, bias):
    torch.manual_seed(1)
    dev, dt = "cuda", torch.bfloat16
    lead = rows if isinstance(rows, tuple) else (rows,)
    tokens = 1
    for r in lead:
        tokens *= r
    assert ops._wgrad_splits(tokens, n_in, n_out) > 1
    x = torch.randn(*lead, n_in, device=dev, dtype=dt, requires_grad=True)
    w = (torch.randn(n_out, n_in, device=dev, dtype=dt) * n_in ** -0.5).requires_grad_()
    b = torch.randn(n_out, device=dev, dtype=dt, requires_grad=True) if bias else None
    dy = torch.randn(*lead, n_out, device=dev, dtype=dt)
    ins = (x, w, b) if bias else (x, w)
    y = ops.linear(x, w, b)
    assert torch.equal(y, F.linear(x, w, b))
    got = torch.autograd.grad(y, ins, dy)
    ref = torch.autograd.grad(F.linear(x, w, b), ins, dy)
    assert torch.equal(got[0], ref[0])                                   # the same GEMM
    # fp32 truth of the weight gradient; both bf16 results round it once (fp32 accumulation, in a different order)
    truth = dy.reshape(-1, n_out).float().t() @ x.detach().reshape(-1, n_in).float()
    tol = 2 ** -8 * truth.abs().max().item()
    assert (got[1].float() - truth).abs().max().item() <= tol
    assert (got[1].float() - truth).abs().max().item() <= 1.05 * (ref[1].float() - truth).abs().max().item() + 1e-6
    if bias:
        torch.testing.assert_close(got[2], ref[2], rtol=2e-2, atol=2e-2 * tokens ** 0.5)


@pytest.mark.gpu
@pytest.mark.parametrize("b,n,dim,n_qkv,n_gate,bias", [(2, 4096, 256, 384, 24, True), (1, 333, 128, 192, 12, False)])
def test_front_end_as_one_node_equals_its_pieces(b, n, dim, n_qkv, n_gate, bias):
    """norm -> (qkv projection, gate logits) as one autograd node (NSA.py:579, 583, 853) against the same three layers run one
    by one in fp32 (the truth) and in bf16 by the library (the yardstick for the rounding)."""
    torch.manual_seed(2)
    dev, dt = "cuda", torch.bfloat16
    inp = torch.randn(b, n, dim, device=dev).to(dt)
    nw = (1 + 0.1 * torch.randn(dim, device=dev)).to(dt)
    wq = (torch.randn(n_qkv, dim, device=dev) * dim ** -0.5).to(dt)
    wg = (torch.randn(n_gate, dim, device=dev) * dim ** -0.5).to(dt)
    bg = torch.randn(n_gate, device=dev).to(dt) if bias else None
    dq = torch.randn(b, n, n_qkv, device=dev).to(dt)
    dl = torch.randn(b, n, n_gate, device=dev).to(dt)

    def pieces(cast):
        ts = [t if t is None else cast(t).detach().requires_grad_() for t in (inp, nw, wq, wg, bg)]
        i_, nw_, wq_, wg_, bg_ = ts
        xn = F.rms_norm(i_, (dim,), nw_, None if cast(inp).dtype == dt else torch.finfo(torch.float32).eps)
        qkv, lg = F.linear(xn, wq_), F.linear(xn, wg_, bg_)
        grads = torch.autograd.grad((qkv, lg), [t for t in ts if t is not None], (cast(dq), cast(dl)))
        return (qkv, lg), grads

    ts = [t if t is None else t.clone().requires_grad_() for t in (inp, nw, wq, wg, bg)]
    outs = ops.normed_projections(ts[0], ts[1], None, ts[2], ts[3], ts[4])
    grads = torch.autograd.grad(outs, [t for t in ts if t is not None], (dq, dl))
    (o32, g32), (o16, g16) = pieces(lambda t: t.float()), pieces(lambda t: t)
    rel = lambda a, r: ((a.float() - r).norm() / r.norm().clamp_min(1e-9)).item()
    for got, want32, want16 in zip(list(outs) + list(grads), list(o32) + list(g32), list(o16) + list(g16)):
        assert got.shape == want32.shape and got.dtype == dt
        assert rel(got, want32) <= max(1.2 * rel(want16, want32), 2e-3), (rel(got, want32), rel(want16, want32))


@pytest.mark.gpu
def test_under_autocast_the_library_layer_runs():
    torch.manual_seed(3)
    x = torch.randn(4096, 64, device="cuda", requires_grad=True)
    w = torch.randn(32, 64, device="cuda", requires_grad=True)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = ops.linear(x, w)
        ref = F.linear(x, w)
    assert y.dtype == torch.bfloat16 and torch.equal(y, ref)
    gx, gw = torch.autograd.grad(y.float().sum(), (x, w))
    assert gx.dtype == torch.float32 and gw.dtype == torch.float32
