from .plan import LayerCall, LayerPlan, ModelParts, ModelPlan, PartPlan
from .qwen2 import build_qwen2

__all__ = ["LayerCall", "LayerPlan", "ModelParts", "ModelPlan", "PartPlan", "build_qwen2"]
