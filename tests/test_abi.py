"""The C-ABI library loads and exports every symbol include/nsa_hip.h declares (no compute)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "nsa_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\bint\s+(nsa_\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from native_sparse_attention_pytorch_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build with python -m native_sparse_attention_pytorch_amd.build"
    L = ctypes.CDLL(_lib.LIB_PATH)
    names = declared_functions()
    assert len(names) >= 5
    for n in names:
        assert hasattr(L, n), f"{n} declared in include/nsa_hip.h but not exported"
    assert _lib.lib().nsa_abi_version() >= 1


def test_plan_rejects_bad_shapes():
    from native_sparse_attention_pytorch_amd import _lib
    d = _lib.SelectDesc()
    d.batch, d.kv_heads, d.group, d.seq, d.num_sel, d.block, d.dim_head, d.causal = 1, 2, 4, 128, 4, 64, 64, 1
    for name in ("q_stride", "k_stride", "v_stride", "o_stride"):
        getattr(d, name)[:] = [128 * 64 * 8, 128 * 64, 64]
    sz = [ctypes.c_size_t() for _ in range(3)]
    L = _lib.lib()
    assert L.nsa_select_workspace_bytes(ctypes.byref(d), *[ctypes.byref(s) for s in sz]) == 0
    assert all(s.value > 0 for s in sz)
    d.dim_head = 48
    assert L.nsa_select_workspace_bytes(ctypes.byref(d), *[ctypes.byref(s) for s in sz]) == -2
    d.dim_head, d.group = 64, 3
    assert L.nsa_select_workspace_bytes(ctypes.byref(d), *[ctypes.byref(s) for s in sz]) == -2
    d.group, d.seq = 4, 0
    assert L.nsa_select_workspace_bytes(ctypes.byref(d), *[ctypes.byref(s) for s in sz]) == -1


def test_cpu_tensors_raise():
    import pytest
    import torch
    from native_sparse_attention_pytorch_amd import native_sparse_attend
    q = torch.randn(1, 2, 32, 64, dtype=torch.bfloat16)
    idx = torch.zeros(1, 2, 32, 1, dtype=torch.long)
    with pytest.raises(RuntimeError):
        native_sparse_attend(q, q, q, 16, idx, idx.bool())
