from . import attention, block, embedding, norm, rope, swiglu  # noqa: F401  (registers the parts)
from .base import Part, build_part, part, register_part, unregister_part

__all__ = ["Part", "build_part", "part", "register_part", "unregister_part"]
