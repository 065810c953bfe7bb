from .layout import SparseLayout
from .matmul import matmul
from .softmax import softmax

__all__ = ["SparseLayout", "matmul", "softmax"]
