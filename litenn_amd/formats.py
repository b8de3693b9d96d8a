"""Block formats and dtype ids shared with the C ABI.

Values are the positional values of LiteNN's enums: QuantizedBlockFormat
(src/LiteNN/Quantization.h:31-62) and DataType (src/LiteNN/DType.h:17-30);
block sizes are GetQuantizedBlockLayout (src/LiteNN/Quantization.h:186-217).
"""
from __future__ import annotations

# QuantizedBlockFormat
Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q8_1, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K, F16, F32 = 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 25, 27
FORMAT_NAMES = {Q4_0: "Q4_0", Q4_1: "Q4_1", Q5_0: "Q5_0", Q5_1: "Q5_1", Q8_0: "Q8_0", Q2_K: "Q2_K", Q3_K: "Q3_K",
                Q4_K: "Q4_K", Q5_K: "Q5_K", Q6_K: "Q6_K", F16: "F16", F32: "F32"}
# every block format is decoded inside the streaming GEMV and the matrix-core GEMM
FAST_FORMATS = (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K, Q3_K, Q4_K, Q5_K, Q6_K)  # streaming GEMV
GEMM_FORMATS = FAST_FORMATS  # and inside the matrix-core GEMM

# DataType
DT_F32, DT_F64, DT_I32, DT_I64, DT_BOOL, DT_F16, DT_BF16, DT_F8E4M3, DT_F8E5M2, DT_I8, DT_U8 = range(11)
DTYPE_SIZE = {DT_F32: 4, DT_F64: 8, DT_I32: 4, DT_I64: 8, DT_BOOL: 1, DT_F16: 2, DT_BF16: 2, DT_F8E4M3: 1,
              DT_F8E5M2: 1, DT_I8: 1, DT_U8: 1}

_LAYOUT = {Q4_0: (32, 18), Q4_1: (32, 20), Q5_0: (32, 22), Q5_1: (32, 24), Q8_0: (32, 34), Q2_K: (256, 84),
           Q3_K: (256, 110), Q4_K: (256, 144), Q5_K: (256, 176), Q6_K: (256, 210), F16: (1, 2), F32: (1, 4)}


def block_layout(fmt: int) -> tuple[int, int]:
    """(elements per block, bytes per block)."""
    try:
        return _LAYOUT[fmt]
    except KeyError:
        raise ValueError(f"unsupported block format {fmt}") from None


def row_bytes(fmt: int, k: int) -> int:
    elems, nbytes = block_layout(fmt)
    if k % elems:
        raise ValueError(f"row width {k} is incompatible with block size {elems}")
    return k // elems * nbytes


def bytes_per_element(fmt: int) -> float:
    elems, nbytes = block_layout(fmt)
    return nbytes / elems
