from . import (attention, block, differential_attention, feedforward, gated_attention, latent_attention,  # noqa: F401
               linear_attention, matrix_memory, norm, parallel, recurrent, retention, rope, routed, side, window_attention)  # noqa: F401  (registers the parts)
from .block import build_block, register_arrangement
from .model import DecoderModel, cache_needs, expected_tensors
from .registry import (PagedKV, PagedLatent, RowState, TensorDecl, build_part, impl_of, register_part,
                       tensors_of)

__all__ = ["DecoderModel", "cache_needs", "expected_tensors", "build_block", "register_arrangement",
           "PagedKV", "PagedLatent", "RowState", "TensorDecl", "build_part", "impl_of", "register_part",
           "tensors_of"]
