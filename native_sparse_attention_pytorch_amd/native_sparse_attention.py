"""Import-path alias: the reference keeps `SparseAttention` in `native_sparse_attention_pytorch/native_sparse_attention.py`
(NSA.py:188); here it lives in `sparse_attention.py`."""
from .sparse_attention import SparseAttention  # noqa: F401
