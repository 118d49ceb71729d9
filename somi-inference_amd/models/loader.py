"""From a model folder (or a configuration and a seed) to a model on the GPU.

Reference: ``load_model`` (somi_inference/models/loader.py:19-29) dispatches on
the configuration and returns the adapter and the config dict; weights come from
a library model's state dict (somi_inference/models/qwen2_adapter.py:228-252).
Here the class is chosen by config.json's architecture through the registry and
the tensors are read from the folder's safetensors by name.
"""

from __future__ import annotations

import os

import torch

from ..cache.manager import CacheManager
from ..config.base import ModelConfig, read_config_json
from ..config.engine import normalize_dtype
from ..config.registry import config_from_dict, resolve_architecture
from ..engine.runner import ModelRunner
from ..parts.base import Runtime
from ..weights.source import RandomSource, SafetensorsSource
from .decoder import DecoderModel

_TORCH_DTYPE = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def make_runtime(dtype: object = "bfloat16", device: str | torch.device = "cuda:0") -> Runtime:
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError(f"the engine runs on the GPU only (device {device} given); there is no CPU path")
    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible; the engine has no CPU path")
    torch.cuda.set_device(device)
    return Runtime(_TORCH_DTYPE[normalize_dtype(dtype)], device)


def load_model(model_dir: str | os.PathLike, dtype: object = "bfloat16",
               device: str | torch.device = "cuda:0") -> tuple[DecoderModel, ModelConfig]:
    """Build the model that ``<model_dir>/config.json`` names and load ``model.safetensors``."""
    arch, config = config_from_dict(read_config_json(model_dir))
    model = DecoderModel(arch.build_plan(config), make_runtime(dtype, device))
    model.load(SafetensorsSource(os.fspath(model_dir)))
    return model, config


def random_model(config: ModelConfig, seed: int, dtype: object = "bfloat16",
                 device: str | torch.device = "cuda:0") -> DecoderModel:
    """A model of seeded random weights drawn on the device (no folder is written)."""
    arch = resolve_architecture(config.architecture)
    model = DecoderModel(arch.build_plan(config), make_runtime(dtype, device))
    model.load(RandomSource(model.weight_specs(), seed))
    return model


def make_runner(model: DecoderModel, *, block_size: int, num_blocks: int, max_requests: int) -> ModelRunner:
    cache = CacheManager(model.cache_needs(), block_size=block_size, num_blocks=num_blocks,
                         max_requests=max_requests, dtype=model.runtime.dtype, device=model.runtime.device)
    return ModelRunner(model, cache)
