"""Model plans and the generic decoder that runs them."""

from .decoder import DecoderModel
from .loader import load_model, make_runner, make_runtime, random_model
from .plan import LayerSpec, ModelPlan, collect_weight_specs
from .qwen2 import qwen2_plan

__all__ = ["DecoderModel", "LayerSpec", "ModelPlan", "collect_weight_specs", "load_model",
           "make_runner", "make_runtime", "qwen2_plan", "random_model"]
