"""What a part says about each of its tensors: shape in the file, role, and how to draw it."""

from __future__ import annotations

from dataclasses import dataclass

MATRIX = "matrix"        # operand of a matrix product: kept in the compute dtype
TABLE = "table"          # rows looked up by index: kept in the compute dtype
VECTOR = "vector"        # bias / norm gain / norm offset: kept in 32-bit
INT_TABLE = "int_table"  # integer table: kept as int32


@dataclass(frozen=True)
class Normal:
    """Draw from N(mean, std)."""

    std: float
    mean: float = 0.0


@dataclass(frozen=True)
class TensorSpec:
    shape: tuple  # as stored in the file
    role: str
    init: Normal
    # Stored [in, out] (the Conv1D layout of GPT-2 files); kept transposed, [out, in], which is
    # what the matrix kernels read.
    keep_transposed: bool = False
