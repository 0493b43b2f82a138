"""ctypes binding of libnsa_hip.so (declarations: include/nsa_hip.h).  There is no fallback:
if the library is missing or a call fails, a RuntimeError is raised."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("NSA_HIP_LIB") or os.path.join(HERE, "libnsa_hip.so")    # NSA_HIP_LIB: load another build of the same ABI

_lib = None


class SelectDesc(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("kv_heads", C.c_int32), ("group", C.c_int32), ("seq", C.c_int32),
        ("num_sel", C.c_int32), ("block", C.c_int32), ("dim_head", C.c_int32), ("causal", C.c_int32),
        ("idx_is_int64", C.c_int32), ("scale", C.c_float),
        ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3), ("o_stride", C.c_int64 * 3),
    ]


class DenseDesc(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("kv_heads", C.c_int32), ("group", C.c_int32), ("seq", C.c_int32),
        ("num_keys", C.c_int32), ("num_mem", C.c_int32), ("dim_head", C.c_int32),
        ("mode", C.c_int32), ("causal", C.c_int32), ("window", C.c_int32), ("stride", C.c_int32),
        ("pool", C.c_int32), ("sel_block", C.c_int32), ("share", C.c_int32), ("scale", C.c_float),
        ("dkv_fp32", C.c_int32),
        ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3),
        ("o_stride", C.c_int64 * 3), ("do_stride", C.c_int64 * 3),
    ]


class DecodeDesc(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("kv_heads", C.c_int32), ("group", C.c_int32), ("dim_head", C.c_int32),
        ("mode", C.c_int32), ("start", C.c_int32), ("count", C.c_int32), ("num_mem", C.c_int32),
        ("block", C.c_int32), ("num_sel", C.c_int32), ("kv_len", C.c_int32),
        ("per_head_sel", C.c_int32), ("idx_is_int64", C.c_int32), ("scale", C.c_float),
        ("q_stride", C.c_int64 * 2), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3),
    ]


class DecodeStepDesc(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("heads", C.c_int32), ("kv_heads", C.c_int32), ("dim_head", C.c_int32),
        ("pos", C.c_int32), ("num_compressed", C.c_int32), ("num_mem", C.c_int32), ("per_block", C.c_int32),
        ("block", C.c_int32), ("num_sel", C.c_int32), ("share", C.c_int32), ("window", C.c_int32), ("scale", C.c_float),
        ("q_stride", C.c_int64 * 2), ("k_stride", C.c_int64 * 2), ("v_stride", C.c_int64 * 2),
        ("kc_stride", C.c_int64 * 3), ("vc_stride", C.c_int64 * 3), ("ck_stride", C.c_int64 * 3), ("cv_stride", C.c_int64 * 3),
        ("krun_stride", C.c_int64 * 2), ("vrun_stride", C.c_int64 * 2),
    ]


class QkvDesc(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("seq", C.c_int32), ("heads", C.c_int32), ("kv_heads", C.c_int32), ("dim_head", C.c_int32),
        ("block", C.c_int32), ("stride", C.c_int32), ("fp32", C.c_int32), ("offset", C.c_int32),
        ("qkv_stride", C.c_int64 * 2),
    ]


_ERR = {-1: "invalid argument", -2: "shape not supported by the compiled kernels", -3: "workspace too small"}


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m native_sparse_attention_pytorch_amd.build` "
                "(hipcc, gfx950).  There is no non-HIP fallback.")
        L = C.CDLL(LIB_PATH)
        vp, sz = C.c_void_p, C.c_size_t
        L.nsa_abi_version.restype = C.c_int
        L.nsa_select_workspace_bytes.argtypes = [C.POINTER(SelectDesc), C.POINTER(sz), C.POINTER(sz), C.POINTER(sz)]
        L.nsa_select_build_index.argtypes = [C.POINTER(SelectDesc), vp, vp, vp, sz, vp]
        L.nsa_select_fwd.argtypes = [C.POINTER(SelectDesc), vp, vp, vp, vp, vp, vp, vp, sz, vp, vp, vp]
        L.nsa_select_bwd.argtypes = [C.POINTER(SelectDesc)] + [vp] * 11 + [sz] + [vp] * 5
        L.nsa_selftest_mfma.argtypes = [vp] * 6
        L.nsa_selftest_mfma.restype = C.c_int
        L.nsa_probe_row_traffic.argtypes = [vp, sz, vp, sz, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_uint32, vp]
        L.nsa_probe_row_traffic.restype = C.c_int
        L.nsa_select_fwd_timed.argtypes = L.nsa_select_fwd.argtypes + [vp, C.c_int]
        L.nsa_select_bwd_timed.argtypes = L.nsa_select_bwd.argtypes + [vp, C.c_int]
        L.nsa_select_fwd_timed.restype = L.nsa_select_bwd_timed.restype = C.c_int
        L.nsa_dense_workspace_bytes.argtypes = [C.POINTER(DenseDesc), C.POINTER(sz)]
        L.nsa_dense_fwd.argtypes = [C.POINTER(DenseDesc)] + [vp] * 7
        L.nsa_dense_bwd.argtypes = [C.POINTER(DenseDesc)] + [vp] * 7 + [sz] + [vp] * 4
        L.nsa_compress_topk_supported.argtypes = [C.POINTER(DenseDesc), C.c_int32]
        L.nsa_compress_topk_fwd.argtypes = [C.POINTER(DenseDesc)] + [vp] * 5 + [C.c_int32, vp, vp, vp]
        L.nsa_compress_topk_supported.restype = L.nsa_compress_topk_fwd.restype = C.c_int
        L.nsa_topk.argtypes = [vp, C.c_int64, C.c_int32, C.c_int32, C.c_int32, vp, vp, vp, vp]
        L.nsa_topk_prefix.argtypes = [vp, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, vp, vp, vp, vp]
        fp = C.POINTER(C.c_float)
        L.nsa_rmsnorm_partials.argtypes = [C.c_int64]
        L.nsa_rmsnorm_fwd.argtypes = [C.c_int64, C.c_int32, vp, C.c_int64, vp, C.c_float, vp, vp, vp]
        L.nsa_rmsnorm_bwd.argtypes = [C.c_int64, C.c_int32, vp, C.c_int64, vp, vp, vp, vp, vp, C.c_int32, vp, vp]
        L.nsa_colsum_workspace.argtypes = [C.c_int64, C.c_int32, C.c_int32]
        L.nsa_colsum_workspace.restype = C.c_int64
        L.nsa_colsum.argtypes = [vp, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int32, vp, C.c_int32, vp, vp]
        L.nsa_sum_slices.argtypes = [vp, C.c_int32, C.c_int64, vp, C.c_int32, vp]
        L.nsa_sum_slices.restype = C.c_int
        L.nsa_rmsnorm_partials.restype = L.nsa_rmsnorm_fwd.restype = L.nsa_rmsnorm_bwd.restype = L.nsa_colsum.restype = C.c_int
        i3 = C.POINTER(C.c_int64)
        L.nsa_gate_fwd.argtypes = [C.c_int32] * 4 + [vp, vp, i3, vp, i3, vp, i3, vp, vp]
        L.nsa_gate_bwd.argtypes = [C.c_int32] * 4 + [vp, vp, i3, vp, i3, vp, i3, vp, vp, vp, vp, vp, vp]
        L.nsa_rope.argtypes = [vp, i3, C.c_int32, C.c_int32, C.c_int32, C.c_int32, vp, C.c_int32, C.c_int32, vp, i3, vp]
        L.nsa_rope.restype = C.c_int
        L.nsa_decode_workspace_bytes.argtypes = [C.POINTER(DecodeDesc), C.POINTER(sz)]
        L.nsa_decode_attend.argtypes = [C.POINTER(DecodeDesc)] + [vp] * 8 + [sz, vp, vp, vp]
        L.nsa_decode_workspace_bytes.restype = L.nsa_decode_attend.restype = C.c_int
        L.nsa_decode_attend_noalloc.argtypes = [C.POINTER(DecodeDesc)] + [vp] * 10
        L.nsa_decode_attend_noalloc.restype = C.c_int
        dd = C.POINTER(DecodeDesc)
        L.nsa_decode_combine.argtypes = [dd, vp, dd, vp, dd, vp, vp, vp, vp]
        i2 = C.POINTER(C.c_int64)
        L.nsa_decode_prep.argtypes = [vp, i2, vp, i2, vp, i2, C.c_int32, C.c_int32, C.c_int32, C.c_int32, vp, C.c_int32, vp, vp, i2, vp, i2, vp, i2, vp, i2, vp]
        L.nsa_decode_combine.restype = L.nsa_decode_prep.restype = C.c_int
        L.nsa_decode_topk.argtypes = [vp] + [C.c_int32] * 7 + [vp, vp, vp, vp]
        L.nsa_decode_topk.restype = C.c_int
        ds = C.POINTER(DecodeStepDesc)
        L.nsa_decode_step_workspace_bytes.argtypes = [ds, C.POINTER(sz), C.POINTER(sz), C.POINTER(sz), C.POINTER(C.c_int32)]
        L.nsa_decode_step.argtypes = [ds] + [vp] * 14 + [sz, vp, vp]
        L.nsa_decode_step_workspace_bytes.restype = L.nsa_decode_step.restype = C.c_int
        L.nsa_decode_step_dyn.argtypes = [ds] + [vp] * 13 + [C.c_int64, C.c_int64, C.c_int32, vp, C.c_int64, vp, vp, sz, vp, C.c_int32, vp]
        L.nsa_decode_step_dyn.restype = C.c_int
        L.nsa_windows_fwd.argtypes = [vp, i3, vp] + [C.c_int32] * 6 + [vp, vp]
        L.nsa_windows_bwd.argtypes = [vp] + [C.c_int32] * 6 + [vp, vp]
        L.nsa_windows_fwd.restype = L.nsa_windows_bwd.restype = C.c_int
        L.nsa_qkv_prep_fwd.argtypes = [C.POINTER(QkvDesc)] + [vp] * 11
        L.nsa_qkv_prep_bwd.argtypes = [C.POINTER(QkvDesc)] + [vp] * 9
        L.nsa_qkv_prep_fwd.restype = L.nsa_qkv_prep_bwd.restype = C.c_int
        L.nsa_dense_fwd_f32.argtypes = [C.POINTER(DenseDesc)] + [vp] * 5 + [C.c_int32, vp]
        L.nsa_select_fwd_f32.argtypes = [C.POINTER(SelectDesc)] + [vp] * 7 + [C.c_int32, C.c_int32, vp]
        L.nsa_dense_fwd_f32.restype = L.nsa_select_fwd_f32.restype = C.c_int
        for name in ("nsa_dense_workspace_bytes", "nsa_dense_fwd", "nsa_dense_bwd", "nsa_topk", "nsa_topk_prefix", "nsa_gate_fwd", "nsa_gate_bwd"):
            getattr(L, name).restype = C.c_int
        for name in ("nsa_select_workspace_bytes", "nsa_select_build_index", "nsa_select_fwd", "nsa_select_bwd"):
            getattr(L, name).restype = C.c_int
        _lib = L
    return _lib


def check(rc: int, what: str):
    if rc == 0:
        return
    if rc < 0:
        raise RuntimeError(f"{what}: {_ERR.get(rc, 'error')} (code {rc})")
    raise RuntimeError(f"{what}: HIP launch failed with hipError_t {rc}")
