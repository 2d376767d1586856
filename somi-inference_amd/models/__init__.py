"""Model plans and the generic decoder that runs them."""

from .decoder import DecoderModel
from .loader import load_model, make_runner, make_runtime, random_model
from .plan import LayerSpec, ModelPlan, collect_weight_specs
from .gizilorn import gizilorn_plan
from .kamedra import kamedra_plan
from .metitar import metitar_plan
from .qwen2 import qwen2_plan
from .rusolorn import rusolorn_plan

__all__ = ["DecoderModel", "LayerSpec", "ModelPlan", "collect_weight_specs", "load_model",
           "gizilorn_plan", "kamedra_plan", "make_runner", "metitar_plan", "make_runtime", "qwen2_plan", "random_model", "rusolorn_plan"]
