from . import attention, block, embedding, mlp, norm, position   # noqa: F401  (registers the parts)
from .registry import part_class, register_part
from .runtime import Runtime
from .spec import BlockSpec, LayerCall, ModelSpec, PartSpec

__all__ = ["part_class", "register_part", "Runtime", "BlockSpec", "LayerCall", "ModelSpec", "PartSpec"]
