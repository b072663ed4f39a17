"""Storage dtypes; numeric values follow DeepLearning/Implementation/Tensor/DataType.h:7-27 of the reference."""
from __future__ import annotations

import enum

import numpy as np


class DataType(enum.IntEnum):
    fp16 = 10
    fp32 = 11
    fp64 = 12
    int8 = 13
    int16 = 14
    int32 = 15
    int64 = 16
    uint8 = 17
    uint16 = 18
    uint32 = 19
    uint64 = 20
    boolean = 21
    fp8_e4m3 = 22
    fp8_e5m2 = 23
    bf16 = 24


_SIZES = {
    DataType.fp16: 2, DataType.fp32: 4, DataType.fp64: 8, DataType.int8: 1, DataType.int16: 2, DataType.int32: 4,
    DataType.int64: 8, DataType.uint8: 1, DataType.uint16: 2, DataType.uint32: 4, DataType.uint64: 8, DataType.boolean: 1,
    DataType.fp8_e4m3: 1, DataType.fp8_e5m2: 1, DataType.bf16: 2,
}

# numpy carrier per storage dtype: bf16 and fp8 have no numpy type and travel as raw unsigned integers
_CARRIERS = {
    DataType.fp16: np.float16, DataType.fp32: np.float32, DataType.fp64: np.float64, DataType.int8: np.int8,
    DataType.int16: np.int16, DataType.int32: np.int32, DataType.int64: np.int64, DataType.uint8: np.uint8,
    DataType.uint16: np.uint16, DataType.uint32: np.uint32, DataType.uint64: np.uint64, DataType.boolean: np.uint8,
    DataType.fp8_e4m3: np.uint8, DataType.fp8_e5m2: np.uint8, DataType.bf16: np.uint16,
}


def size_of(dtype: DataType) -> int:
    return _SIZES[DataType(dtype)]


def numpy_carrier(dtype: DataType):
    return np.dtype(_CARRIERS[DataType(dtype)])
