"""Element types of the path, mirroring the reference's DType for the block formats it covers
(core/DType.java:36-98) with the ggml ids GGUF files store (gguf/GgmlType.java:27-65)."""
from __future__ import annotations

from enum import Enum


class DType(Enum):
    #        ggml id, values per block, bytes per block
    F32 = (0, 0, 0)
    I32 = (26, 0, 0)
    Q4_0 = (2, 32, 18)
    Q4_1 = (3, 32, 20)
    Q8_0 = (8, 32, 34)
    Q4_K = (12, 256, 144)
    Q5_K = (13, 256, 176)
    Q6_K = (14, 256, 210)
    # the other block formats the reference dequantises (core/kernels/GgufKernels.java:147-198): bit-exact dequantiser and
    # a plain GEMV, no tuned kernels
    Q5_0 = (6, 32, 22)
    Q5_1 = (7, 32, 24)
    Q2_K = (10, 256, 84)
    Q3_K = (11, 256, 110)

    @property
    def ggml_id(self) -> int:
        return self.value[0]

    def block_values(self) -> int:
        return self.value[1]

    def block_bytes(self) -> int:
        return self.value[2]

    def is_block_quantized(self) -> bool:
        return self.value[1] > 0

    @staticmethod
    def from_ggml_id(i: int) -> "DType":
        for t in DType:
            if t.ggml_id == i:
                return t
        raise ValueError(f"ggml type id {i} has no tensor type on this path")
