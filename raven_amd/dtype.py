"""The dtype table: tags, storage types and classes.

Tags equal Nx's ``Dtype.Packed.tag`` and the reference C backend's enum
(packages/nx/lib/backend_c/nx_c.h:130-200); the storage column is how a host
buffer holds one element (packages/nx/lib/buffer/nx_buffer_stubs.h:18-25):
bf16 and fp8 travel as raw bit patterns, bool as a 0/1 byte, int4/uint4 packed
two per byte with the low nibble first.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np


@dataclass(frozen=True)
class DType:
    name: str
    tag: int
    np_storage: np.dtype  # numpy dtype of the host storage array
    itemsize: int  # bytes per element, 0 for packed nibbles
    cls: str  # "float" | "sint" | "uint" | "complex" | "bool"
    packed: bool = False

    def __repr__(self) -> str:  # pragma: no cover - cosmetic
        return f"nx.{self.name}"

    @property
    def is_float(self) -> bool:
        return self.cls == "float"

    @property
    def is_int(self) -> bool:
        return self.cls in ("sint", "uint")

    @property
    def is_complex(self) -> bool:
        return self.cls == "complex"

    @property
    def is_bool(self) -> bool:
        return self.cls == "bool"

    def nbytes(self, count: int) -> int:
        """Bytes of ``count`` contiguous elements (nx_c.h:325-328)."""
        if self.packed:
            return (count + 1) // 2
        return count * self.itemsize


def _d(name, tag, np_t, size, cls, packed=False):
    return DType(name, tag, np.dtype(np_t), size, cls, packed)


float16 = _d("float16", 0, np.float16, 2, "float")
float32 = _d("float32", 1, np.float32, 4, "float")
float64 = _d("float64", 2, np.float64, 8, "float")
bfloat16 = _d("bfloat16", 3, np.uint16, 2, "float")
float8_e4m3 = _d("float8_e4m3", 4, np.uint8, 1, "float")
float8_e5m2 = _d("float8_e5m2", 5, np.uint8, 1, "float")
int4 = _d("int4", 6, np.uint8, 0, "sint", packed=True)
uint4 = _d("uint4", 7, np.uint8, 0, "uint", packed=True)
int8 = _d("int8", 8, np.int8, 1, "sint")
uint8 = _d("uint8", 9, np.uint8, 1, "uint")
int16 = _d("int16", 10, np.int16, 2, "sint")
uint16 = _d("uint16", 11, np.uint16, 2, "uint")
int32 = _d("int32", 12, np.int32, 4, "sint")
uint32 = _d("uint32", 13, np.uint32, 4, "uint")
int64 = _d("int64", 14, np.int64, 8, "sint")
uint64 = _d("uint64", 15, np.uint64, 8, "uint")
complex64 = _d("complex64", 16, np.complex64, 8, "complex")
complex128 = _d("complex128", 17, np.complex128, 16, "complex")
bool_ = _d("bool", 18, np.uint8, 1, "bool")

ALL = [
    float16, float32, float64, bfloat16, float8_e4m3, float8_e5m2, int4, uint4,
    int8, uint8, int16, uint16, int32, uint32, int64, uint64, complex64,
    complex128, bool_,
]
BY_TAG = {d.tag: d for d in ALL}
BY_NAME = {d.name: d for d in ALL}
COMPUTE = [d for d in ALL if not d.packed]


def of_tag(tag: int) -> DType:
    return BY_TAG[tag]
