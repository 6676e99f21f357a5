from . import qwen2_moe  # registers Qwen2MoeForCausalLM
from .spec import LayerCall, ModelSpec

__all__ = ["LayerCall", "ModelSpec", "qwen2_moe"]
