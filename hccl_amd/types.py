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


# the enumerators under their short names, so that `from hccl_amd import types as T; T.BFP16, T.SUM` reads like the
# C header's HCCL_DATA_TYPE_BFP16 / HCCL_REDUCE_SUM
INT8, INT16, INT32, FP16, FP32, INT64, UINT64, UINT8, UINT16, UINT32, FP64, BFP16, INT128 = (
    int(DataType.INT8), int(DataType.INT16), int(DataType.INT32), int(DataType.FP16), int(DataType.FP32),
    int(DataType.INT64), int(DataType.UINT64), int(DataType.UINT8), int(DataType.UINT16), int(DataType.UINT32),
    int(DataType.FP64), int(DataType.BFP16), int(DataType.INT128))
SUM, PROD, MAX, MIN = int(ReduceOp.SUM), int(ReduceOp.PROD), int(ReduceOp.MAX), int(ReduceOp.MIN)
