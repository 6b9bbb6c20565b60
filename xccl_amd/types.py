"""Enums of the mem-component boundary; values are ABI (include/xccl_rocm_types.h,
reference src/api/xccl.h:371-407, src/api/xccl_status.h:10-30)."""
import enum


class Status(enum.IntEnum):
    OK = 0
    INPROGRESS = 1
    ERR_NO_MESSAGE = -1
    ERR_NO_RESOURCE = -2
    ERR_NO_MEMORY = -4
    ERR_INVALID_PARAM = -5
    ERR_UNREACHABLE = -6
    ERR_NOT_IMPLEMENTED = -8
    ERR_MESSAGE_TRUNCATED = -9
    ERR_NO_PROGRESS = -10
    ERR_BUFFER_TOO_SMALL = -11
    ERR_NO_ELEM = -12
    ERR_UNSUPPORTED = -22
    ERR_LAST = -100


class Op(enum.IntEnum):
    MAX = 0
    MIN = 1
    SUM = 2
    PROD = 3
    AND = 4
    OR = 5
    XOR = 6
    LAND = 7
    LOR = 8
    LXOR = 9
    BAND = 10
    BOR = 11
    BXOR = 12
    MAXLOC = 13
    MINLOC = 14
    LAST_PREDEFINED = 15
    UNSUPPORTED = 16


class Dt(enum.IntEnum):
    INT8 = 0
    INT16 = 1
    INT32 = 2
    INT64 = 3
    INT128 = 4
    UINT8 = 5
    UINT16 = 6
    UINT32 = 7
    UINT64 = 8
    UINT128 = 9
    FLOAT16 = 10
    FLOAT32 = 11
    FLOAT64 = 12
    LAST_PREDEFINED = 13
    UNSUPPORTED = 14


class MemType(enum.IntEnum):
    """ucs_memory_type_t of UCX v1.10."""
    HOST = 0
    CUDA = 1
    CUDA_MANAGED = 2
    ROCM = 3
    ROCM_MANAGED = 4
    LAST = 5


class StreamType(enum.IntEnum):
    CUDA = 0
    ROCM = 1


_DT_SIZE = {
    Dt.INT8: 1, Dt.UINT8: 1,
    Dt.INT16: 2, Dt.UINT16: 2, Dt.FLOAT16: 2,
    Dt.INT32: 4, Dt.UINT32: 4, Dt.FLOAT32: 4,
    Dt.INT64: 8, Dt.UINT64: 8, Dt.FLOAT64: 8,
    Dt.INT128: 16, Dt.UINT128: 16,
}


def dt_size(dt) -> int:
    """xccl_dt_size (reference src/api/xccl.h:478-502): bytes per element, 0 if unknown."""
    try:
        return _DT_SIZE.get(Dt(int(dt)), 0)
    except ValueError:
        return 0


INT_DTYPES = (Dt.INT8, Dt.INT16, Dt.INT32, Dt.INT64, Dt.UINT8, Dt.UINT16, Dt.UINT32, Dt.UINT64)
FP_DTYPES = (Dt.FLOAT16, Dt.FLOAT32, Dt.FLOAT64)
INT_OPS = (Op.MAX, Op.MIN, Op.SUM, Op.PROD, Op.LAND, Op.LOR, Op.LXOR, Op.BAND, Op.BOR, Op.BXOR)
FP_OPS = (Op.MAX, Op.MIN, Op.SUM, Op.PROD)


def supported_pairs():
    """Every (dtype, op) the component has a kernel for."""
    return [(d, o) for d in INT_DTYPES for o in INT_OPS] + [(d, o) for d in FP_DTYPES for o in FP_OPS]
