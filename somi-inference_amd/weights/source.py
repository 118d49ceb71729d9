"""Where tensors come from: a model folder, or a seeded generator.

Both answer the same three questions (which names, what shape and stored
dtype, give me this tensor on that device), so the loader validates and
places them the same way.
"""

from __future__ import annotations

import hashlib
import json
import os

import torch

from .safetensors_io import SafetensorsError, TensorEntry, read_header, read_tensor
from .spec import MATRIX, TABLE, VECTOR, WeightSpec


class WeightSource:
    def names(self) -> list[str]:
        raise NotImplementedError

    def shape(self, name: str) -> tuple[int, ...]:
        raise NotImplementedError

    def stored_dtype(self, name: str) -> torch.dtype:
        raise NotImplementedError

    def read(self, name: str, device: torch.device | str) -> torch.Tensor:
        """The tensor in its stored dtype on ``device``."""
        raise NotImplementedError


class SafetensorsSource(WeightSource):
    """``model.safetensors`` of a model folder, or the shards its index file names."""

    def __init__(self, model_dir: str) -> None:
        self.model_dir = os.fspath(model_dir)
        single = os.path.join(self.model_dir, "model.safetensors")
        index = os.path.join(self.model_dir, "model.safetensors.index.json")
        self._entries: dict[str, TensorEntry] = {}
        if os.path.isfile(single):
            self._entries = read_header(single)
        elif os.path.isfile(index):
            with open(index, "r", encoding="utf-8") as handle:
                weight_map = json.load(handle).get("weight_map", {})
            for shard in sorted(set(weight_map.values())):
                header = read_header(os.path.join(self.model_dir, shard))
                for name, entry in header.items():
                    if weight_map.get(name) == shard:
                        self._entries[name] = entry
            lost = sorted(set(weight_map) - set(self._entries))
            if lost:
                raise SafetensorsError(f"{index}: tensors named by the index but absent from their shard: {lost[:8]}")
        else:
            raise SafetensorsError(
                f"{self.model_dir}: neither model.safetensors nor model.safetensors.index.json found")

    def names(self) -> list[str]:
        return list(self._entries)

    def shape(self, name: str) -> tuple[int, ...]:
        return self._entries[name].shape

    def stored_dtype(self, name: str) -> torch.dtype:
        return self._entries[name].dtype

    def read(self, name: str, device: torch.device | str) -> torch.Tensor:
        return read_tensor(self._entries[name]).to(device)


def tensor_seed(seed: int, name: str) -> int:
    """A 63-bit seed that depends on (seed, tensor name) only, so any tensor
    can be generated alone and in any order."""
    digest = hashlib.sha256(f"{int(seed)}:{name}".encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensor(spec: WeightSpec, seed: int, device: torch.device | str,
                  float_dtype: torch.dtype) -> torch.Tensor:
    """N(mean, std) drawn in float32 from the tensor's own generator, then rounded once.

    The stream of a generator differs between the CPU and the GPU, so a folder
    written on the CPU and tensors made on the GPU from the same seed are
    different (equally valid) models.
    """
    device = torch.device(device)
    gen = torch.Generator(device=device)
    gen.manual_seed(tensor_seed(seed, spec.name))
    if spec.role == TABLE:
        return torch.randint(0, 2**15, spec.shape, generator=gen, device=device, dtype=torch.int32)
    out = torch.randn(spec.shape, generator=gen, device=device, dtype=torch.float32)
    out.mul_(spec.init.std).add_(spec.init.mean)
    return out.to(float_dtype)


HOST_DRAW_ELEMENTS = 1 << 28      # models of up to this many weights are drawn on the host by default


class RandomSource(WeightSource):
    """Seeded random tensors made on demand (no file).

    ``draw_on``: "host" draws with the host's generator, so the tensors equal those that
    :func:`~somi_inference_amd.weights.write_random_model` writes for the same seed (a plain implementation can
    read the same model from a folder); "device" draws on the target device without a host copy, which is what
    models of tens of gigabytes need, and gives another (equally valid) model for the same seed.  "auto" takes
    the host up to HOST_DRAW_ELEMENTS weights in all.
    """

    def __init__(self, specs: list[WeightSpec], seed: int, stored: torch.dtype = torch.bfloat16,
                 draw_on: str = "auto") -> None:
        self._specs = {s.name: s for s in specs}
        self.seed = int(seed)
        self.stored = stored
        if draw_on not in ("auto", "host", "device"):
            raise ValueError(f"draw_on must be auto, host or device, got {draw_on!r}")
        if draw_on == "auto":
            total = 0
            for s in specs:
                count = 1
                for dim in s.shape:
                    count *= int(dim)
                total += count
            draw_on = "host" if total <= HOST_DRAW_ELEMENTS else "device"
        self.draw_on = draw_on

    def names(self) -> list[str]:
        return list(self._specs)

    def shape(self, name: str) -> tuple[int, ...]:
        return self._specs[name].shape

    def stored_dtype(self, name: str) -> torch.dtype:
        return torch.int32 if self._specs[name].role == TABLE else self.stored

    def read(self, name: str, device: torch.device | str) -> torch.Tensor:
        if self.draw_on == "host":
            return random_tensor(self._specs[name], self.seed, "cpu", self.stored).to(device)
        return random_tensor(self._specs[name], self.seed, device, self.stored)


__all__ = ["MATRIX", "VECTOR", "TABLE", "RandomSource", "SafetensorsSource", "WeightSource",
           "random_tensor", "tensor_seed"]
