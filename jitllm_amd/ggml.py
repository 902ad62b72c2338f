"""GGUF block geometry of the weight representations on the path.

Mirrors ``GGMLType`` of the reference (src/main/java/org/beehive/jitllm/format/GGMLType.java:7,13,
18-20,27-29): a type is (elements per block, bytes per block); a ``[d x n]`` weight is ``d`` rows of
``n / block_elems`` blocks each, row-major, exactly as the file stores them.  The integer values
are ggml's type ids, the ones a GGUF tensor-info record carries.
"""
from __future__ import annotations

import enum


class GGMLType(enum.IntEnum):
    Q4_0 = 2
    Q4_1 = 3    # plain single-token projection and the decode-once batched path
    Q5_0 = 6    # likewise
    Q8_0 = 8
    Q4_K = 12
    Q5_K = 13   # plain single-token projection and the decode-once batched path
    Q6_K = 14   # likewise
    IQ4_XS = 23  # likewise

    @property
    def block_elems(self) -> int:
        return _GEOMETRY[self][0]

    @property
    def block_bytes(self) -> int:
        return _GEOMETRY[self][1]

    def byte_size_for(self, number_of_elements: int) -> int:
        """GGMLType.byteSizeFor (GGMLType.java:81-85)."""
        if number_of_elements % self.block_elems:
            raise ValueError(
                f"{number_of_elements} elements is not a whole number of {self.name} blocks")
        return number_of_elements // self.block_elems * self.block_bytes

    def row_bytes(self, n: int) -> int:
        return self.byte_size_for(n)


_GEOMETRY = {
    GGMLType.Q4_0: (32, 18),
    GGMLType.Q4_1: (32, 20),
    GGMLType.Q5_0: (32, 22),
    GGMLType.IQ4_XS: (256, 136),
    GGMLType.Q8_0: (32, 34),
    GGMLType.Q4_K: (256, 144),
    GGMLType.Q5_K: (256, 176),
    GGMLType.Q6_K: (256, 210),
}
