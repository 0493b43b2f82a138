"""RMS norm (NSA.py:230, 579) and the column sums of the backward pass, HIP kernels through the C ABI against the closed form
y = x / sqrt(mean(x^2) + eps) * w evaluated in fp64 (and its autograd), and against plain fp64 sums."""
import ctypes as C

import pytest
import torch

from native_sparse_attention_pytorch_amd import _lib, ops

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def closed_form(x, w, eps):
    x, w = x.double(), w.double()
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


@pytest.mark.parametrize("shape", [(4, 512, 1024), (3, 8), (1, 4096), (37, 520), (1030, 2048), (2, 5, 7, 64), (1024, 256)])
@pytest.mark.parametrize("eps", [None, 1e-5])
def test_rms_norm_forward_backward(shape, eps):
    torch.manual_seed(sum(shape))
    x = (torch.randn(*shape, device="cuda") * 2 + 0.3).to(BF).requires_grad_()
    w = (1 + 0.2 * torch.randn(shape[-1], device="cuda")).to(BF).requires_grad_()
    dy = torch.randn(*shape, device="cuda").to(BF)
    assert ops.rms_norm_supported(x, w)
    e = torch.finfo(torch.float32).eps if eps is None else eps          # None: the epsilon of the fp32 the norm is computed in
    y = ops.rms_norm(x, w, eps)
    xd, wd = x.detach().double().cpu().requires_grad_(), w.detach().double().cpu().requires_grad_()
    yr = closed_form(xd, wd, e)
    # one rounding of the fp32 result to bf16: 2^-8 relative
    assert ((y.double().cpu() - yr).abs() <= 2 ** -8 * yr.abs() + 1e-6).all()
    dx, dw = torch.autograd.grad(y, (x, w), dy)
    dxr, dwr = torch.autograd.grad(yr, (xd, wd), dy.double().cpu())
    assert ((dx.double().cpu() - dxr).abs() <= 2 ** -8 * dxr.abs() + 2e-5 * dxr.abs().max()).all()
    assert ((dw.double().cpu() - dwr).abs() <= 2 ** -8 * dwr.abs() + 2e-5 * dwr.abs().max()).all()
    # the library's own norm (what nn.RMSNorm runs): never closer to the closed form than this kernel - a different epsilon
    # for eps=None (2^-7, the bf16 one, shifts every value by 0.4 %) or a dropped factor would show here
    yt = torch.nn.functional.rms_norm(x, x.shape[-1:], w, eps)
    rms = lambda t: (t.double().cpu() - yr).pow(2).mean().sqrt().item()
    assert rms(y) <= 1.02 * rms(yt) + 1e-12
    assert ((y.float() - yt.float()).abs() <= 2 ** -7 * yt.float().abs() + 1e-6).all()


def test_rms_norm_reads_strided_rows_and_is_deterministic():
    torch.manual_seed(0)
    big = torch.randn(300, 1536, device="cuda").to(BF)
    x = big[:, 256:256 + 1024]
    w = torch.randn(1024, device="cuda").to(BF)
    y = ops.rms_norm(x, w)
    assert torch.equal(y, ops.rms_norm(x.contiguous(), w))
    xg, wg = x.clone().requires_grad_(), w.clone().requires_grad_()
    dy = torch.randn(300, 1024, device="cuda").to(BF)
    a = torch.autograd.grad(ops.rms_norm(xg, wg), (xg, wg), dy)
    b = torch.autograd.grad(ops.rms_norm(xg, wg), (xg, wg), dy)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_rms_norm_limits_through_the_abi():
    L = _lib.lib()
    x = torch.zeros(4, 4104, device="cuda", dtype=BF)
    r = torch.zeros(4, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    assert L.nsa_rmsnorm_fwd(4, 4104, p(x), 4104, p(x), 1e-5, p(x), p(r), None) == -2          # dim above 4096
    assert L.nsa_rmsnorm_fwd(4, 12, p(x), 12, p(x), 1e-5, p(x), p(r), None) == -2              # dim not a multiple of 8
    assert L.nsa_rmsnorm_fwd(4, 64, p(x), 60, p(x), 1e-5, p(x), p(r), None) == -2              # rows overlap
    assert L.nsa_rmsnorm_fwd(-1, 64, p(x), 64, p(x), 1e-5, p(x), p(r), None) == -1
    assert L.nsa_rmsnorm_fwd(0, 64, None, 64, None, 1e-5, None, None, None) == 0               # nothing to do
    assert L.nsa_rmsnorm_bwd(4, 64, p(x), 64, p(x), p(r), p(x), p(x), p(x), 0, None, None) == -1   # weight gradient without scratch
    assert not ops.rms_norm_supported(x, x[0])
    # the wrapper falls back to the library for what the kernel does not take
    xf = torch.randn(4, 12, device="cuda")
    wf = torch.randn(12, device="cuda")
    assert torch.equal(ops.rms_norm(xf, wf, 1e-6), torch.nn.functional.rms_norm(xf, (12,), wf, 1e-6))


@pytest.mark.parametrize("rows,cols", [(16384, 48), (4080, 2048), (4080, 64), (1, 8), (7, 4096), (100000, 8), (513, 2056)])
def test_colsum(rows, cols):
    torch.manual_seed(rows + cols)
    x = torch.randn(rows, cols, device="cuda").to(BF)
    truth = x.double().sum(0)
    scale = x.double().abs().sum(0)
    got = ops.colsum(x, torch.float32)
    assert ((got.double() - truth).abs() <= 1e-6 * scale + 1e-30).all()           # fp32 additions of exact inputs
    got16 = ops.colsum(x)
    assert got16.dtype == BF
    assert ((got16.double() - truth).abs() <= 2 ** -8 * truth.abs() + 1e-6 * scale).all()
    assert torch.equal(got, ops.colsum(x, torch.float32))                          # fixed order of additions


def test_colsum_leading_axes_and_strided_rows():
    torch.manual_seed(5)
    big = torch.randn(6, 50, 96, device="cuda").to(BF)
    x = big[..., 16:80]
    got = ops.colsum(x, torch.float32)
    torch.testing.assert_close(got.double(), x.double().sum((0, 1)), rtol=1e-6, atol=1e-4)


@pytest.mark.parametrize("b,h,w,j,d", [(4, 4, 255, 32, 64), (1, 2, 1, 4, 8), (2, 3, 17, 8, 128)])
def test_window_position_grad(b, h, w, j, d):
    torch.manual_seed(b * w)
    dwin = torch.randn(b, h, w, j, d, device="cuda").to(BF)
    got = ops.window_position_grad(dwin, torch.float32)
    truth = dwin.double().sum((0, 2))
    assert got.shape == (h, j, d)
    assert ((got.double() - truth).abs() <= 1e-6 * dwin.double().abs().sum((0, 2)) + 1e-30).all()


def test_colsum_limits_through_the_abi():
    L = _lib.lib()
    x = torch.ones(4, 16, device="cuda", dtype=BF)
    out = torch.full((16,), 7.0, device="cuda")
    ws = torch.zeros(1024, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    assert L.nsa_colsum(p(x), 1, 0, 1, 0, 4, 16, 12, p(out), 1, p(ws), None) == -2             # cols not a multiple of 8
    assert L.nsa_colsum(p(x), 1, 0, 1, 0, 4, 12, 16, p(out), 1, p(ws), None) == -2             # row stride not a multiple of 8
    assert L.nsa_colsum(p(x), 0, 0, 1, 0, 4, 16, 16, p(out), 1, p(ws), None) == -1
    assert L.nsa_colsum(p(x), 1, 0, 1, 0, 4, 16, 16, p(out), 1, None, None) == -1              # no workspace
    assert L.nsa_colsum(None, 1, 0, 1, 0, 0, 16, 16, p(out), 1, None, None) == 0               # no rows: zeros
    torch.cuda.synchronize()
    assert torch.equal(out, torch.zeros_like(out))
    assert L.nsa_colsum(p(x), 1, 0, 1, 0, 4, 16, 16, p(out), 1, p(ws), None) == 0
    torch.cuda.synchronize()
    assert torch.equal(out, torch.full_like(out, 4.0))
    assert L.nsa_colsum_workspace(4, 16, 1) >= 4 * 16


@pytest.mark.parametrize("parts,shape,out_dtype", [(8, (1024, 1024), BF), (8, (48, 1024), BF), (4, (64, 2048), torch.float32), (1, (4, 4), BF),
                                                   (7, (33, 12), BF)])
def test_sum_slices(parts, shape, out_dtype):
    torch.manual_seed(parts)
    L = _lib.lib()
    sl = torch.randn(parts, *shape, device="cuda")
    out = torch.empty(shape, device="cuda", dtype=out_dtype)
    n = shape[0] * shape[1]
    assert L.nsa_sum_slices(C.c_void_p(sl.data_ptr()), parts, n, C.c_void_p(out.data_ptr()), int(out_dtype == torch.float32), None) == 0
    torch.cuda.synchronize()
    truth = sl.double().sum(0)
    tol = (1e-6 if out_dtype == torch.float32 else 2 ** -8) * truth.abs() + 1e-6 * sl.double().abs().sum(0)
    assert ((out.double() - truth).abs() <= tol).all()
    assert L.nsa_sum_slices(C.c_void_p(sl.data_ptr()), parts, 6, C.c_void_p(out.data_ptr()), 0, None) == -2      # n not a multiple of 4
    assert L.nsa_sum_slices(C.c_void_p(sl.data_ptr()), 0, n, C.c_void_p(out.data_ptr()), 0, None) == -1
