from .layout import SparseLayout
from .matmul import matmul
from .softmax import softmax
from .attention import attention

__all__ = ["SparseLayout", "matmul", "softmax", "attention"]
