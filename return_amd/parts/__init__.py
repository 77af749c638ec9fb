from . import attention, block, conv, delta, embedding, mix, mlp, moe, norm, passes, position, share, side, ssm   # noqa: F401  (registers the parts)
from .registry import part_class, register_part
from .runtime import Runtime
from .spec import BlockSpec, LayerCall, ModelSpec, PartSpec

__all__ = ["part_class", "register_part", "Runtime", "BlockSpec", "LayerCall", "ModelSpec", "PartSpec"]
