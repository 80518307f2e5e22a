"""What a part says about each tensor it needs: name, shape, role and how to make a
random one.  The loader checks files against these; the random-weights mode fills them."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

# roles
MATRIX = "matrix"    # a linear map [out, in]; kept in the run's compute dtype
VECTOR = "vector"    # norm weights, biases, conv taps: consumed in 32-bit arithmetic
TABLE = "table"      # rows looked up by integer id (embeddings); compute dtype

# random initialisation kinds
INIT_NORMAL = "normal"             # N(0, matrix_std)
INIT_ONES = "ones"                 # 1, or 1 + N(0, norm_jitter) when jitter is asked for
INIT_SMALL = "small"               # N(0, matrix_std), for biases


@dataclass(frozen=True)
class TensorSpec:
    name: str
    shape: Tuple[int, ...]
    role: str = MATRIX
    init: str = INIT_NORMAL

    def numel(self) -> int:
        n = 1
        for s in self.shape:
            n *= s
        return n
