"""MI355X-native (gfx950 HIP) implementation of the Native Sparse Attention hot path."""
from .ops import native_sparse_attend  # noqa: F401
