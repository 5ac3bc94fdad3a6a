"""ggml tensor types and block geometry (src/ml/gguf/reader.cr:34-98, 119-127)."""
import enum


class TensorType(enum.IntEnum):
    F32 = 0
    F16 = 1
    Q4_0 = 2
    Q4_1 = 3
    Q5_0 = 6
    Q5_1 = 7
    Q8_0 = 8
    Q2_K = 10
    Q3_K = 11
    Q4_K = 12
    Q5_K = 13
    Q6_K = 14
    Q8_K = 15
    IQ4_NL = 20

    @property
    def block_bytes(self):
        return _BLOCK_BYTES[self]

    @property
    def block_elements(self):
        return _BLOCK_ELEMENTS[self]

    def data_bytes(self, n_elements):
        """TensorInfo#data_bytes for n_elements of this type."""
        if self in (TensorType.F32, TensorType.F16):
            return n_elements * self.block_bytes
        return ((n_elements + self.block_elements - 1) // self.block_elements) * self.block_bytes


_BLOCK_BYTES = {
    TensorType.F32: 4, TensorType.F16: 2, TensorType.Q4_0: 18, TensorType.Q4_1: 20, TensorType.Q5_0: 22,
    TensorType.Q5_1: 24, TensorType.Q8_0: 34, TensorType.Q2_K: 84, TensorType.Q3_K: 110, TensorType.Q4_K: 144,
    TensorType.Q5_K: 176, TensorType.Q6_K: 210, TensorType.Q8_K: 292, TensorType.IQ4_NL: 18,
}
_BLOCK_ELEMENTS = {
    TensorType.F32: 1, TensorType.F16: 1, TensorType.Q4_0: 32, TensorType.Q4_1: 32, TensorType.Q5_0: 32,
    TensorType.Q5_1: 32, TensorType.Q8_0: 32, TensorType.Q2_K: 256, TensorType.Q3_K: 256, TensorType.Q4_K: 256,
    TensorType.Q5_K: 256, TensorType.Q6_K: 256, TensorType.Q8_K: 256, TensorType.IQ4_NL: 32,
}
