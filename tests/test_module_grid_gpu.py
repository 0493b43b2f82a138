"""The reference's own parametrisation grid (tests/test_sparse_attn.py:9-17) on the HIP module,
complete (selection blocks of 8, 16 and 32; the reference's Triton path stops at 16), and checked
numerically against the CPU oracle instead of by shape only: causal /
non-causal, ragged and tiny sequences, no selectable block, num_selected_blocks = 0, per-head
selection, differentiable top-k, MHA and GQA."""
import itertools

import pytest
import torch

from oracle import nsa_oracle as O
from tests.util import assert_close, capture_selection

pytestmark = pytest.mark.gpu
DEV = "cuda"

GRID = list(itertools.product(
    (False, True),            # use_diff_topk
    (False, True),            # causal
    (1, 4, 31, 32, 120),      # seq_len
    (8, 4),                   # kv_heads
    (8, 16, 32),              # selection_block_size
    (8, 4),                   # compress_block_size
    (2, 4),                   # compress_block_sliding_stride
    (0, 2),                   # num_selected_blocks
    (False, True),            # query_heads_share_selected_kv
))


def _case(diff, causal, n, kvh, B, cbs, st, S, share, seed):
    from native_sparse_attention_pytorch_amd import ops
    from native_sparse_attention_pytorch_amd.sparse_attention import SparseAttention
    kw = dict(dim=128, dim_head=64, heads=8, kv_heads=kvh, causal=causal, sliding_window_size=2, selection_block_size=B,
              compress_block_size=cbs, compress_block_sliding_stride=st, num_selected_blocks=S, use_diff_topk=diff,
              query_heads_share_selected_kv=share)
    torch.manual_seed(seed)
    ref = O.SparseAttentionOracle(**kw)
    with torch.no_grad():
        ref.to_strategy_combine[0].weight.normal_(std=0.05)
        ref.compress_mem_kv.normal_(std=0.5)
        for p in ref.parameters():
            p.copy_(p.to(torch.bfloat16).float())
    mod = SparseAttention(**kw)
    mod.load_state_dict(ref.state_dict(), strict=True)
    mod = mod.to(DEV).to(torch.bfloat16)
    x = torch.randn(2, n, 128, generator=torch.Generator().manual_seed(seed + 1)).to(torch.bfloat16)
    captured = {}
    with capture_selection(captured):
        out = mod(x.to(DEV))
    assert out.shape == x.shape
    want = ref(x.float(), selection_override=captured.get("sel"))
    assert_close(out, want, 3e-2 * want.abs().max().item() + 1e-3, 2e-2, f"case {kw} n={n}")


@pytest.mark.parametrize("chunk", range(8))
def test_reference_grid_against_oracle(chunk):
    cases = GRID[chunk::8]          # 240 of the 1920 grid points per test
    for k, c in enumerate(cases):
        print("grid case", c, flush=True)
        _case(*c, seed=chunk * 1000 + k)
