"""MI355X-native (gfx950 HIP) implementation of the Native Sparse Attention hot path."""
from .ops import (compress_attend, gate_combine, importance_topk, native_sparse_attend,  # noqa: F401
                  sliding_attend)
from .sparse_attention import SparseAttention  # noqa: F401
