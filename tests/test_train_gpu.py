"""Training-step harness (BASELINE config 5): the HIP-backed Transformer's loss sequence against
the CPU oracle transformer - live on a reduced size, and against the committed oracle fixture
(tests/golden/train_cfg5_oracle_losses.json) at the full config-5 size."""
import json
import os

import pytest
import torch

from oracle import nsa_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda"
HERE = os.path.dirname(os.path.abspath(__file__))


def _run_product(cfg, ids, seed, steps, lr):
    from native_sparse_attention_pytorch_amd.transformer import Transformer
    torch.manual_seed(seed)
    model = Transformer(**cfg).to(DEV)            # fp32 master weights, bf16 compute via autocast
    opt = torch.optim.Adam(model.parameters(), lr=lr)
    ids = ids.to(DEV)
    losses = []
    for _ in range(steps):
        with torch.autocast("cuda", dtype=torch.bfloat16):
            loss = model(ids, return_loss=True)
        loss.backward()
        opt.step()
        opt.zero_grad()
        losses.append(loss.item())
    return losses


def test_train_small_matches_live_oracle():
    cfg = dict(num_tokens=256, dim=128, depth=2, dim_head=64, heads=4, kv_heads=2,
               sparse_attn_kwargs=dict(sliding_window_size=32, compress_block_size=16, compress_block_sliding_stride=8,
                                       selection_block_size=16, num_selected_blocks=4))
    seed, steps, lr = 3, 10, 1e-3
    ids = torch.randint(0, 256, (2, 257), generator=torch.Generator().manual_seed(4))
    torch.manual_seed(seed)
    ref = O.TransformerOracle(**cfg)
    opt = torch.optim.Adam(ref.parameters(), lr=lr)
    want = []
    for _ in range(steps):
        loss = ref(ids, return_loss=True)
        loss.backward()
        opt.step()
        opt.zero_grad()
        want.append(loss.item())
    got = _run_product(cfg, ids, seed, steps, lr)
    print("oracle", want)
    print("hip   ", got)
    assert want[-1] < want[0] - 0.05, "the oracle run must actually learn, or the comparison pins nothing"
    # measured agreement is a few 1e-5 per step (bf16 autocast against the fp32 oracle); the loss falls by ~0.07 per step, so a
    # bound of 2e-3 tells a wrong layer from rounding
    for a, b in zip(got, want):
        assert abs(a - b) < 2e-3, (got, want)


def test_train_config5_matches_oracle_fixture():
    path = os.path.join(HERE, "golden", "train_cfg5_oracle_losses.json")
    fx = json.load(open(path))
    ids = torch.randint(0, 256, (fx["batch"], fx["seq"] + 1), generator=torch.Generator().manual_seed(fx["seed"] + 1))
    got = _run_product(fx["config"], ids, fx["seed"], fx["steps"], fx["lr"])
    print("oracle fixture", fx["losses"])
    print("hip           ", got)
    for a, b in zip(got, fx["losses"]):
        assert abs(a - b) < 2e-3, (got, fx["losses"])


def test_train_config5_with_fp32_masters_matches_oracle_fixture():
    """The same ten steps with the model itself in bf16 and the optimizer on fp32 master weights (training.Fp32Masters)
    instead of autocast: the same arithmetic without the per-layer casts, the same bound."""
    from native_sparse_attention_pytorch_amd.transformer import Transformer
    from native_sparse_attention_pytorch_amd.training import Fp32Masters
    fx = json.load(open(os.path.join(HERE, "golden", "train_cfg5_oracle_losses.json")))
    ids = torch.randint(0, 256, (fx["batch"], fx["seq"] + 1), generator=torch.Generator().manual_seed(fx["seed"] + 1)).to(DEV)
    torch.manual_seed(fx["seed"])
    model = Transformer(**fx["config"]).to(DEV)
    mw = Fp32Masters(model)
    opt = torch.optim.Adam(mw.masters, lr=fx["lr"])
    got = []
    for _ in range(fx["steps"]):
        loss = model(ids, return_loss=True)
        loss.backward()
        mw.step(opt)
        got.append(loss.item())
    print("oracle fixture", fx["losses"])
    print("hip, masters  ", got)
    for a, b in zip(got, fx["losses"]):
        assert abs(a - b) < 2e-3, (got, fx["losses"])


def _small_model():
    from native_sparse_attention_pytorch_amd.transformer import Transformer
    torch.manual_seed(5)
    return Transformer(num_tokens=256, dim=256, depth=3, dim_head=64, heads=4, kv_heads=2,
                       sparse_attn_kwargs=dict(sliding_window_size=32, compress_block_size=16, compress_block_sliding_stride=8,
                                               selection_block_size=16, num_selected_blocks=4)).to(DEV)


def test_graphed_step_equals_the_launched_step_on_every_replay():
    """training.GraphedStep: forward + backward replayed from one HIP graph.  Every replay - different tokens each time, the
    same step launched normally and a synchronisation in between - must give the launched step's loss and gradients.  (A graph
    that contains the library's multi-block sums gives the first replay right and later ones wrong on this platform: bias
    gradients of 1e37.  While recording, those sums are this library's kernels instead.)"""
    from native_sparse_attention_pytorch_amd.training import Fp32Masters, GraphedStep
    model = _small_model()
    Fp32Masters(model)                                    # bf16 model
    params = list(model.parameters())
    names = [n for n, _ in model.named_parameters()]
    data = [torch.randint(0, 256, (4, 513), device=DEV, generator=torch.Generator(device=DEV).manual_seed(i)) for i in range(7)]
    step = GraphedStep(model, data[0])
    assert sum(g is not None for g in step.grads) >= len(params) - 8
    for rep, ids in enumerate(data):
        for p in params:
            p.grad = None
        want_loss = model(ids, return_loss=True)
        want_loss.backward()
        want = [None if p.grad is None else p.grad.clone() for p in params]
        torch.cuda.synchronize()
        loss = step(ids)
        torch.cuda.synchronize()
        assert abs(loss.item() - want_loss.item()) < 1e-5, (rep, loss.item(), want_loss.item())
        for n, p, w in zip(names, params, want):
            assert (p.grad is None) == (w is None), n
            if w is not None:
                assert torch.isfinite(p.grad).all(), f"replay {rep}: non-finite gradient of {n}"
                err = (p.grad.float() - w.float()).abs().max().item()
                # identical kernels on identical inputs; only the bias sums take another kernel while recording (fp32 sums of
                # bf16 values in another order: within one bf16 rounding of the result)
                tol = 1e-2 * max(w.float().abs().max().item(), 1e-6) if n.endswith("bias") else 0.0
                assert err <= tol, f"replay {rep}: gradient of {n} differs by {err} (largest entry {w.float().abs().max().item()})"


def test_train_config5_graphed_with_fp32_masters_matches_oracle_fixture():
    """Ten Adam steps with forward + backward replayed from a graph and the optimizer on fp32 masters outside it: the loss
    sequence of the oracle fixture, to the bound of the launched step."""
    from native_sparse_attention_pytorch_amd.transformer import Transformer
    from native_sparse_attention_pytorch_amd.training import Fp32Masters, GraphedStep
    fx = json.load(open(os.path.join(HERE, "golden", "train_cfg5_oracle_losses.json")))
    ids = torch.randint(0, 256, (fx["batch"], fx["seq"] + 1), generator=torch.Generator().manual_seed(fx["seed"] + 1)).to(DEV)
    torch.manual_seed(fx["seed"])
    model = Transformer(**fx["config"]).to(DEV)
    mw = Fp32Masters(model)
    opt = torch.optim.Adam(mw.masters, lr=fx["lr"])
    step = GraphedStep(model, ids)
    got = []
    for _ in range(fx["steps"]):
        got.append(step(ids).item())
        mw.step(opt)
    print("oracle fixture", fx["losses"])
    print("graphed       ", got)
    for a, b in zip(got, fx["losses"]):
        assert abs(a - b) < 2e-3, (got, fx["losses"])


def test_graphed_step_refuses_a_model_that_was_already_stepped():
    """Recording after normally launched training steps of the same model is not supported (it ended the process on this
    platform); the helper says so instead of starting the recording."""
    from native_sparse_attention_pytorch_amd.training import Fp32Masters, GraphedStep
    model = _small_model()
    Fp32Masters(model)
    ids = torch.randint(0, 256, (2, 257), device=DEV)
    model(ids, return_loss=True).backward()
    with pytest.raises(RuntimeError, match="before the model's first"):
        GraphedStep(model, ids)


def test_graphed_step_refuses_fp32_parameters():
    from native_sparse_attention_pytorch_amd.training import GraphedStep
    model = _small_model()                                # fp32 parameters: would train under autocast
    with pytest.raises(RuntimeError, match="bf16 model"):
        GraphedStep(model, torch.randint(0, 256, (2, 257), device=DEV))


def test_graphed_step_of_a_bare_attention_module():
    """GraphedStep with a loss function of its own: one SparseAttention layer, float inputs instead of token ids."""
    from native_sparse_attention_pytorch_amd import SparseAttention
    from native_sparse_attention_pytorch_amd.training import GraphedStep
    torch.manual_seed(9)
    attn = SparseAttention(dim=256, dim_head=64, heads=4, kv_heads=2, sliding_window_size=32, compress_block_size=16,
                           compress_block_sliding_stride=8, selection_block_size=16, num_selected_blocks=4).to(DEV).bfloat16()
    w = torch.randn(2, 384, 256, device=DEV, dtype=torch.bfloat16)
    loss_fn = lambda m, x: (m(x).float() * w.float()).mean()
    xs = [torch.randn(2, 384, 256, device=DEV, dtype=torch.bfloat16, generator=torch.Generator(device=DEV).manual_seed(i)) for i in range(4)]
    step = GraphedStep(attn, xs[0], loss_fn=loss_fn)
    params = list(attn.parameters())
    names = [n for n, _ in attn.named_parameters()]
    for rep, x in enumerate(xs):
        for p in params:
            p.grad = None
        want_loss = loss_fn(attn, x)
        want_loss.backward()
        want = [None if p.grad is None else p.grad.clone() for p in params]
        torch.cuda.synchronize()
        loss = step(x)
        torch.cuda.synchronize()
        assert abs(loss.item() - want_loss.item()) <= 1e-6 * max(1.0, abs(want_loss.item())), (rep, loss.item(), want_loss.item())
        for n, p, wg in zip(names, params, want):
            assert (p.grad is None) == (wg is None), n
            if wg is not None:
                err = (p.grad.float() - wg.float()).abs().max().item()
                tol = 1e-2 * max(wg.float().abs().max().item(), 1e-6) if n.endswith("bias") else 0.0
                assert torch.isfinite(p.grad).all() and err <= tol, f"replay {rep}: gradient of {n} differs by {err}"
