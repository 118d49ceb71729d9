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
                 device: str | torch.device = "cuda:0", draw_on: str = "auto") -> DecoderModel:
    """A model of seeded random weights (no folder is written).  Small models are drawn on the host and equal what
    ``write_random_model`` writes for the seed; large ones are drawn on the device (see ``RandomSource``)."""
    arch = resolve_architecture(config.architecture)
    model = DecoderModel(arch.build_plan(config), make_runtime(dtype, device))
    model.load(RandomSource(model.weight_specs(), seed, draw_on=draw_on))
    return model


def pages_that_fit(model: DecoderModel, block_size: int, memory_fraction: float = 0.9) -> int:
    """How many cache pages per group fit into ``memory_fraction`` of the device memory that is free now (after
    the weights): the pool of a GPU with hundreds of gigabytes is sized by its memory, not by a constant."""
    if not 0.0 < memory_fraction <= 1.0:
        raise ValueError(f"memory_fraction must be in (0, 1], got {memory_fraction}")
    per_page = CacheManager.page_bytes(model.cache_needs(), block_size, model.runtime.dtype)
    if per_page == 0:
        return 1
    free, _ = torch.cuda.mem_get_info(model.runtime.device)
    pages = int(free * memory_fraction) // per_page
    if pages < 1:
        raise RuntimeError(f"no cache page of {per_page} bytes fits into {memory_fraction:.2f} of the {free} free bytes")
    return pages


def make_runner(model: DecoderModel, *, block_size: int, num_blocks: int | None, max_requests: int,
                memory_fraction: float = 0.9) -> ModelRunner:
    """``num_blocks=None``: as many pages as fit into ``memory_fraction`` of the free device memory."""
    if num_blocks is None:
        num_blocks = pages_that_fit(model, block_size, memory_fraction)
    cache = CacheManager(model.cache_needs(), block_size=block_size, num_blocks=num_blocks,
                         max_requests=max_requests, dtype=model.runtime.dtype, device=model.runtime.device)
    return ModelRunner(model, cache)
