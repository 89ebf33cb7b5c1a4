"""dtype table: float32 only, as in dlgrad/dtype.py:8-27.

`CDataPtr` in the reference is cffi's CData; here a pointer is whatever the
device runtime hands out (a `DevicePtr` for HIP), so the alias is `object`.
"""
from __future__ import annotations

from enum import Enum, auto
from typing import Any

CDataPtr = Any
Scalar = float


class DType(Enum):
    FLOAT32 = auto()

    @staticmethod
    def from_str(d: str) -> "DType":
        try:
            return DType[d.upper()]
        except KeyError:
            raise ValueError(f"Invalid dtype: {d}") from None

    @staticmethod
    def get_n_bytes(d: "DType") -> int:
        return _NBYTES[d]


_NBYTES = {DType.FLOAT32: 4}
