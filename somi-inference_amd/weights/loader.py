"""Checks a weight source against what the model's parts declare, then places tensors.

The reference relies on ``load_state_dict(strict=True)``
(somi_inference/models/qwen2_adapter.py:251) for missing/unexpected keys and
shape mismatches, skips ``lm_head.weight`` and anything with ``rotary_emb`` in
its name (:161-166).  Here the check is explicit and raises one
:class:`WeightMismatchError` that lists every missing tensor, every unexpected
tensor and every wrong shape at once.
"""

from __future__ import annotations

import fnmatch
from typing import Iterable

import torch

from .source import WeightSource
from .spec import MATRIX, TABLE, VECTOR, WeightSpec


class WeightMismatchError(ValueError):
    """The source's tensors do not match what the model declares."""

    def __init__(self, missing: list[str], unexpected: list[str],
                 wrong_shape: list[tuple[str, tuple, tuple]],
                 wrong_kind: list[tuple[str, str, str]]) -> None:
        self.missing = missing
        self.unexpected = unexpected
        self.wrong_shape = wrong_shape
        self.wrong_kind = wrong_kind
        lines = ["model weights do not match the configuration:"]
        if missing:
            lines.append(f"  missing tensors ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected tensors ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong_shape:
            lines.append(f"  wrong shapes ({len(wrong_shape)}): " + "; ".join(
                f"{n}: file has {tuple(got)}, configuration needs {tuple(want)}"
                for n, got, want in wrong_shape))
        if wrong_kind:
            lines.append(f"  wrong dtypes ({len(wrong_kind)}): " + "; ".join(
                f"{n}: file has {got}, needs {want}" for n, got, want in wrong_kind))
        super().__init__("\n".join(lines))


def check_weights(specs: Iterable[WeightSpec], source: WeightSource,
                  ignore: Iterable[str] = ()) -> None:
    """Raise :class:`WeightMismatchError` unless names, shapes and kinds agree.

    ``ignore`` holds glob patterns of tensors that may be present without
    being used (computed buffers, a head that is tied away).
    """
    specs = list(specs)
    wanted = {s.name: s for s in specs}
    present = set(source.names())
    patterns = list(ignore)
    missing = sorted(n for n in wanted if n not in present)
    unexpected = sorted(n for n in present if n not in wanted
                        and not any(fnmatch.fnmatchcase(n, p) for p in patterns))
    wrong_shape, wrong_kind = [], []
    for name, spec in wanted.items():
        if name not in present:
            continue
        if tuple(source.shape(name)) != spec.shape:
            wrong_shape.append((name, tuple(source.shape(name)), spec.shape))
        stored = source.stored_dtype(name)
        if spec.role == TABLE and stored.is_floating_point:
            wrong_kind.append((name, str(stored), "an integer type"))
        if spec.role != TABLE and not stored.is_floating_point:
            wrong_kind.append((name, str(stored), "a floating-point type"))
    if missing or unexpected or wrong_shape or wrong_kind:
        raise WeightMismatchError(missing, unexpected, wrong_shape, wrong_kind)


def device_dtype(role: str, compute: torch.dtype) -> torch.dtype:
    """The dtype a tensor of this role is held in on the device.

    Matrix operands take the compute dtype (a bfloat16 checkpoint stays
    bfloat16 in the bfloat16 engine and widens exactly in the float32 one).
    Scales and biases are always float32: widening a bfloat16 value is exact,
    and one stored in 32-bit stays 32-bit.  Integer tables are int32.
    """
    if role == MATRIX:
        return compute
    if role == VECTOR:
        return torch.float32
    return torch.int32


class WeightFetcher:
    """Hands each declared tensor to the part that asked for it, on the device,
    in the dtype its role gives.  Built after :func:`check_weights` passed."""

    def __init__(self, specs: Iterable[WeightSpec], source: WeightSource,
                 compute: torch.dtype, device: torch.device | str) -> None:
        self._specs = {s.name: s for s in specs}
        self._source = source
        self._compute = compute
        self._device = torch.device(device)
        self.fetched: set[str] = set()

    def __call__(self, name: str) -> torch.Tensor:
        spec = self._specs[name]
        tensor = self._source.read(name, self._device)
        self.fetched.add(name)
        return tensor.to(device_dtype(spec.role, self._compute)).contiguous()
