from . import attention, block, ends, mlp, norm, rope  # noqa: F401  (they register themselves)
from .model import DecoderModel, build_blocks, expected_tensors
from .registry import PartError, build_part, part_class, register_part

__all__ = ["DecoderModel", "build_blocks", "expected_tensors", "PartError", "build_part", "part_class",
           "register_part"]
