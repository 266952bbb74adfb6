from . import attention, block, feedforward, norm, rope  # noqa: F401  (registers the parts)
from .block import build_block, register_arrangement
from .model import DecoderModel, cache_needs, expected_tensors
from .registry import (PagedKV, RowState, TensorDecl, build_part, impl_of, register_part,
                       tensors_of)

__all__ = ["DecoderModel", "cache_needs", "expected_tensors", "build_block", "register_arrangement",
           "PagedKV", "RowState", "TensorDecl", "build_part", "impl_of", "register_part",
           "tensors_of"]
