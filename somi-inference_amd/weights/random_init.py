"""Random-weights mode: a model folder from a configuration and a seed.

The reference has no such mode; its tests lean on the default initialisation
of library modules (tests/models/test_qwen2_adapter.py:38-39).  Here the
model's parts declare their tensors (name, shape, distribution) and this
module draws each from a generator keyed by (seed, tensor name).
"""

from __future__ import annotations

import json
import os

import torch

from ..config.base import ModelConfig
from ..config.registry import resolve_architecture
from .safetensors_io import write_file
from .source import random_tensor
from .spec import TABLE


def write_random_model(model_dir: str, config: ModelConfig, seed: int,
                       stored: torch.dtype = torch.bfloat16) -> str:
    """Write ``config.json`` and ``model.safetensors`` for ``config``; returns the folder.

    Floating-point tensors are drawn in float32 and stored in ``stored``
    (bfloat16 by default, as checkpoints of this architecture are), so the
    bfloat16 engine, the float32 engine and a plain implementation all read
    exactly the same values.
    """
    from ..models.plan import collect_weight_specs  # late: models imports weights

    arch = resolve_architecture(config.architecture)
    plan = arch.build_plan(config)
    specs = collect_weight_specs(plan)
    os.makedirs(model_dir, exist_ok=True)
    tensors = {}
    for spec in specs:
        tensors[spec.name] = random_tensor(spec, seed, "cpu", stored)
    write_file(os.path.join(model_dir, "model.safetensors"), tensors,
               metadata={"format": "pt", "seed": str(seed)})
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(config.to_dict(), handle, indent=2)
        handle.write("\n")
    return model_dir
