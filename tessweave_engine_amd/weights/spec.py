"""What a part says about each checkpoint tensor it owns."""
from __future__ import annotations

from dataclasses import dataclass

# Roles decide the precision a tensor is held in on the device:
#   matrix  - linear and embedding weights: the compute dtype (bfloat16 or float32)
#   vector  - norm weights and biases: always float32. A tensor stored in 32-bit
#             keeps every bit; one stored in bfloat16 widens exactly.
#   table   - integer tables: int32
MATRIX, VECTOR, TABLE = "matrix", "vector", "table"

# Initialisations of the random-weights mode.
NORMAL, ONE_PLUS_NORMAL = "normal", "one_plus_normal"


@dataclass(frozen=True)
class TensorSpec:
    name: str                 # the safetensors key
    shape: tuple
    role: str = MATRIX
    init: str = NORMAL        # how the random-weights mode draws it
    optional_alias_of: str | None = None   # tied tensors: accepted in a checkpoint, never required

    def __post_init__(self):
        object.__setattr__(self, "shape", tuple(int(s) for s in self.shape))
