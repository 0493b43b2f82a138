"""GroupedMLP (compress_networks.py:73-101, per-head MLP as one batched GEMM per layer) on the device against the
reference's own formulation - two einops mixing layers - holding the same parameters: forward and backward, fp32
(both are fp32 GEMMs: 1e-4) and bf16 (inputs and parameters rounded once, compared with the fp32 result)."""
import pytest
import torch

from tests.test_module_gpu import EinMixGroupedMLP
from tests.util import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("heads,d,cbs,expand,b,w", [(4, 64, 32, 1.0, 2, 37), (2, 128, 16, 0.5, 1, 200), (3, 64, 5, 1.0, 2, 11)])
def test_grouped_mlp_matches_einops_mix_layers_on_device(heads, d, cbs, expand, b, w):
    from native_sparse_attention_pytorch_amd.compress_networks import GroupedMLP
    torch.manual_seed(heads + cbs)
    mine = GroupedMLP(dim_head=d, compress_window_size=cbs, heads=heads, expand_factor=expand).to(DEV)
    lib = EinMixGroupedMLP(dim_head=d, compress_window_size=cbs, heads=heads, expand_factor=expand).to(DEV)
    lib.load_state_dict(mine.state_dict(), strict=True)
    kv = torch.randn(b, heads, w, cbs, d, device=DEV)
    do = torch.randn(b, heads, w, d, device=DEV)
    x1, x2 = kv.clone().requires_grad_(), kv.clone().requires_grad_()
    y1, y2 = mine(x1), lib(x2)
    (y1 * do).sum().backward()
    (y2 * do).sum().backward()
    scale = y2.abs().max().item()
    assert_close(y1, y2, 1e-4 * scale, 1e-4, "fp32 forward")
    assert_close(x1.grad, x2.grad, 1e-4 * x2.grad.abs().max().item(), 1e-4, "fp32 input grad")
    for (n1, p1), (_, p2) in zip(mine.named_parameters(), lib.named_parameters()):
        assert_close(p1.grad, p2.grad, 1e-4 * p2.grad.abs().max().item(), 1e-4, "fp32 grad " + n1)
    # bf16 module, as the attention module runs it
    m16 = GroupedMLP(dim_head=d, compress_window_size=cbs, heads=heads, expand_factor=expand).to(DEV)
    m16.load_state_dict(mine.state_dict())
    m16 = m16.bfloat16()
    x3 = kv.bfloat16().requires_grad_()
    y3 = m16(x3)
    (y3.float() * do).sum().backward()
    assert_close(y3, y2, 2e-2 * scale, 1e-2, "bf16 forward")
    for (n1, p3), (_, p2) in zip(m16.named_parameters(), lib.named_parameters()):
        e = ((p3.grad.float() - p2.grad).norm() / p2.grad.norm()).item()
        assert e < 5e-2, f"bf16 grad {n1}: {e:.4f}"
