"""DataType and Status with the reference's integer values (include/axono/core/types.h:18-27,54-64;
Python enums at axono/python/src/nanobind_module.cpp:185-203)."""
from enum import IntEnum

import numpy as np


class DataType(IntEnum):
    INT8 = 0
    INT16 = 1
    INT32 = 2
    INT64 = 3
    FLOAT16 = 4
    FLOAT32 = 5
    FLOAT64 = 6
    BOOLEAN = 7


class Status(IntEnum):
    OK = 0
    INVALID_ARGUMENT = 1
    OUT_OF_MEMORY = 2
    UNSUPPORTED_TYPE = 3
    SHAPE_MISMATCH = 4
    INTERNAL_ERROR = 5
    DEVICE_ERROR = 6
    INVALID_PTR = 7
    DEVICE_MISMATCH = 8


DTYPE_SIZE = {
    DataType.INT8: 1, DataType.INT16: 2, DataType.INT32: 4, DataType.INT64: 8,
    DataType.FLOAT16: 2, DataType.FLOAT32: 4, DataType.FLOAT64: 8, DataType.BOOLEAN: 1,
}

DTYPE_TO_NUMPY = {
    DataType.INT8: np.int8, DataType.INT16: np.int16, DataType.INT32: np.int32, DataType.INT64: np.int64,
    DataType.FLOAT16: np.float16, DataType.FLOAT32: np.float32, DataType.FLOAT64: np.float64,
    DataType.BOOLEAN: np.bool_,
}

NUMPY_TO_DTYPE = {np.dtype(v): k for k, v in DTYPE_TO_NUMPY.items()}
