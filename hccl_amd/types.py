"""Enumerations of include/hccl_types.h."""
import enum


class Result(enum.IntEnum):
    SUCCESS = 0
    E_PARA = 1
    E_PTR = 2
    E_MEMORY = 3
    E_INTERNAL = 4
    E_NOT_SUPPORT = 5
    E_NOT_FOUND = 6
    E_UNAVAIL = 7
    E_RUNTIME = 15
    E_SUSPENDING = 22


class DataType(enum.IntEnum):
    INT8 = 0
    INT16 = 1
    INT32 = 2
    FP16 = 3
    FP32 = 4
    INT64 = 5
    UINT64 = 6
    UINT8 = 7
    UINT16 = 8
    UINT32 = 9
    FP64 = 10
    BFP16 = 11
    INT128 = 12


class ReduceOp(enum.IntEnum):
    SUM = 0
    PROD = 1
    MAX = 2
    MIN = 3


_SIZES = [1, 2, 4, 2, 4, 8, 8, 1, 2, 4, 8, 2, 16, 2, 1, 1, 1, 1]


def dtype_size(dt):
    return _SIZES[int(dt)]
