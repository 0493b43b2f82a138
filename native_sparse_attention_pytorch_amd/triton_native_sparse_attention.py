"""Import-path alias: the reference exposes the selection-attention operator as
`native_sparse_attention_pytorch.triton_native_sparse_attention.native_sparse_attend` (TRI.py:1938-1987); the operator
of the same name and signature here runs the HIP kernels (`ops.native_sparse_attend`)."""
from .ops import native_sparse_attend  # noqa: F401
