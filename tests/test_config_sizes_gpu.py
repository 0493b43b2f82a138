"""The two named workloads that the other GPU tests only reach at other sizes, at their exact shapes:

  * selection attention, b1 n8192 16/4 heads d64 B64, 15 selected + own block: backward.  The upstream gradient is
    non-zero only on a few query blocks, so the oracle run on those queries yields every gradient of the whole problem.
  * the full SparseAttention module, b4 n4096 dim1024 16/4 heads d64 window 512, compress 32/16, B64, 16 selected,
    forward + backward (NSA.py:549-867 end to end).  Batch elements are independent, so the fp32 oracle runs batch
    element 0 (under the HIP path's block selection); the other three are covered by size-independent properties:
    the module on one batch element alone reproduces its rows of the batched run, and the parameter gradients of the
    batched run are the sum of the four single-element runs.
Bounds as everywhere: forward 2e-2 abs + 1e-2 rel, gradients 5e-2 rel."""
import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import assert_close, assert_grad_close, capture_selection, causal_random_selection

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rand(shape, g, scale):
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def test_config2_selection_backward():
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    b, hq, hk, n, d, B, S = 1, 16, 4, 8192, 64, 64, 15
    g = torch.Generator().manual_seed(2)
    q, k, v = _rand((b, hq, n, d), g, d ** -0.25), _rand((b, hk, n, d), g, d ** -0.25), _rand((b, hk, n, d), g, 1.0)
    idx, msk = causal_random_selection(b, hk, n, B, S, seed=22)
    blocks = [0, 3, 15, 16, 64, 100, 126, 127]
    do = torch.zeros(b, hq, n, d, dtype=torch.bfloat16)
    for w in blocks:
        do[:, :, w * B:(w + 1) * B] = _rand((b, hq, B, d), g, 1.0)
    print("config 2 backward: oracle on", len(blocks), "query blocks", flush=True)
    kr, vr = k.float().requires_grad_(), v.float().requires_grad_()
    loss, ref = 0.0, {}
    for w in blocks:
        sl = slice(w * B, (w + 1) * B)
        qr = q[:, :, sl].float().requires_grad_()
        o = O.select_attend(qr, kr, vr, idx[:, :, sl], msk[:, :, sl], B, causal=True, q_offset=w * B)
        loss = loss + (o * do[:, :, sl].float()).sum()
        ref[w] = (qr, o.detach())
    loss.backward()
    qg, kg, vg = (t.to(DEV).requires_grad_() for t in (q, k, v))
    out = native_sparse_attend(qg, kg, vg, B, idx.to(DEV), msk.to(DEV))
    (out.float() * do.to(DEV).float()).sum().backward()
    torch.cuda.synchronize()
    dq = qg.grad.cpu()
    live = torch.zeros(n, dtype=torch.bool)
    dq_scale = max(r[0].grad.abs().max().item() for r in ref.values())
    for w in blocks:
        sl = slice(w * B, (w + 1) * B)
        live[sl] = True
        assert_close(out[:, :, sl], ref[w][1], 2e-2, 1e-2, f"out, query block {w}")
        assert_close(dq[:, :, sl], ref[w][0].grad, 2e-2 * dq_scale, 5e-2, f"dq, query block {w}")
    assert (dq[:, :, ~live] == 0).all()
    for name, got, want in (("dk", kg.grad, kr.grad), ("dv", vg.grad, vr.grad)):
        e = ((got.float().cpu() - want).norm() / want.norm()).item()
        assert e < 5e-2, f"{name}: rel err {e:.4f}"
        assert_grad_close(got, want, name)


def test_config3_full_module_forward_backward():
    from native_sparse_attention_pytorch_amd import ops
    from native_sparse_attention_pytorch_amd.sparse_attention import SparseAttention
    kw = dict(dim=1024, dim_head=64, heads=16, kv_heads=4, sliding_window_size=512, compress_block_size=32,
              compress_block_sliding_stride=16, selection_block_size=64, num_selected_blocks=16, causal=True)
    b, n = 4, 4096
    torch.manual_seed(3)
    ref = O.SparseAttentionOracle(**kw)
    with torch.no_grad():                        # every branch and parameter matters; values exactly representable in bf16
        ref.to_strategy_combine[0].weight.normal_(std=0.02)
        ref.compress_mem_kv.normal_(std=0.5)
        ref.k_intrablock_positions.normal_(std=0.2)
        ref.v_intrablock_positions.normal_(std=0.2)
        for p in ref.v_compress.parameters():
            p.add_(torch.randn_like(p) * 0.01)
        for p in ref.parameters():
            p.copy_(p.to(torch.bfloat16).float())
    mod = SparseAttention(**kw)
    mod.load_state_dict(ref.state_dict(), strict=True)
    mod = mod.to(DEV).to(torch.bfloat16)
    g = torch.Generator().manual_seed(33)
    x = torch.randn(b, n, kw["dim"], generator=g).to(torch.bfloat16)
    do = torch.randn(b, n, kw["dim"], generator=g).to(torch.bfloat16)

    captured = {}

    def run(xs, dos):
        for p in mod.parameters():
            p.grad = None
        xg = xs.to(DEV).requires_grad_()
        with capture_selection(captured):
            out = mod(xg)
            (out.float() * dos.to(DEV).float()).sum().backward()
            torch.cuda.synchronize()
        grads = {name: p.grad.float().cpu() for name, p in mod.named_parameters() if p.grad is not None}
        return out.detach().cpu(), xg.grad.cpu(), grads, captured["sel"]

    print("config 3: batched HIP run", flush=True)
    out4, dx4, grads4, _ = run(x, do)
    assert out4.shape == x.shape and torch.isfinite(out4.float()).all() and torch.isfinite(dx4.float()).all()

    # --- properties over all four batch elements: independence and additivity
    singles = []
    for e in range(b):
        o1, dx1, g1, sel1 = run(x[e:e + 1], do[e:e + 1])
        singles.append((g1, sel1))
        # equal up to the GEMM library choosing another kernel for another row count (an ulp of bf16) and, through
        # that, a flipped near-tie of the block selection in a handful of rows
        for what, one, four in (("forward", o1, out4[e:e + 1]), ("input grad", dx1, dx4[e:e + 1])):
            tol = 1e-2 * four.float().abs().max().item()
            off = ((one.float() - four.float()).abs().amax(dim=-1) > tol).float().mean().item()
            assert off < 2e-3, f"batch element {e}: {what} of the single run differs from the batched run in {off:.4f} of the rows"
    for name, gsum in grads4.items():
        parts = sum(s[0][name] for s in singles)
        e = ((gsum - parts).norm() / parts.norm().clamp_min(1e-6)).item()
        assert e < 2e-2, f"grad of {name}: batched run vs sum of single runs {e:.4f}"

    # --- batch element 0 against the fp32 oracle under the HIP path's selection
    print("config 3: oracle on batch element 0", flush=True)
    g0, (idx0, live0) = singles[0]
    xr = x[0:1].float().requires_grad_()
    _, parts = ref(xr.detach(), return_parts=True)
    olive = parts["vals"] > 1e-10
    agree = total = 0
    for a, la, o, lo in zip(idx0.flatten(0, 2)[::7], live0.flatten(0, 2)[::7], parts["idx"].flatten(0, 2)[::7], olive.flatten(0, 2)[::7]):
        sa, so = set(a[la].tolist()), set(o[lo].tolist())
        agree += len(sa & so)
        total += max(len(sa), len(so))
    assert agree / max(total, 1) > 0.97, f"selected-block agreement {agree}/{total}"
    want = ref(xr, selection_override=(idx0, live0))
    (want * do[0:1].float()).sum().backward()
    assert_close(out4[0:1], want, 2e-2, 1e-2, "module out, batch element 0")
    e = ((dx4[0:1].float() - xr.grad).norm() / xr.grad.norm()).item()
    assert e < 5e-2, f"input grad rel err {e:.4f}"
    worst = {}
    for name, pr in ref.named_parameters():
        if pr.grad is None:
            continue
        worst[name] = ((g0[name] - pr.grad).norm() / pr.grad.norm().clamp_min(1e-6)).item()
    print("config 3 parameter gradient errors:", {k_: round(v_, 4) for k_, v_ in worst.items()}, flush=True)
    bad = {k_: v_ for k_, v_ in worst.items() if v_ >= 5e-2}
    assert not bad, f"parameter gradients beyond 5e-2: {bad}"
