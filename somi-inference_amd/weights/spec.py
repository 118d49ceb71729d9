"""What a part declares about each tensor it needs."""

from __future__ import annotations

from dataclasses import dataclass

MATRIX = "matrix"   # operand of a matrix product: held in the engine's compute dtype
VECTOR = "vector"   # norm scale or bias: held in float32 (a 32-bit stored tensor stays 32-bit)
TABLE = "table"     # integer table: held as int32


@dataclass(frozen=True)
class Init:
    """Distribution of a tensor in random-weights mode: N(mean, std)."""

    mean: float = 0.0
    std: float = 0.02


@dataclass(frozen=True)
class WeightSpec:
    name: str                   # full tensor name as in the checkpoint
    shape: tuple[int, ...]
    role: str = MATRIX
    init: Init = Init()

    def __post_init__(self) -> None:
        if self.role not in (MATRIX, VECTOR, TABLE):
            raise ValueError(f"weight {self.name!r}: unknown role {self.role!r}")
        object.__setattr__(self, "shape", tuple(int(s) for s in self.shape))
