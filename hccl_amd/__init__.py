"""hccl_amd: HCCL's collective hot path for N virtual ranks in one MI355X's HBM.

The work is done by libhccl_amd.so (hand-written HIP for gfx950).  This package is the Python
binding of its C ABI, used by the tests and the benchmark."""
from . import _lib  # noqa: F401
from .types import DataType, ReduceOp, Result, dtype_size  # noqa: F401
