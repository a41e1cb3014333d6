"""kinetics_amd -- block top-k sparse paged decode attention on MI355X (gfx950).

Hand-written HIP kernels behind a C ABI (include/kinetics_amd.h), exposed as
tensor-level functions (``kinetics_amd.ops``), ``torch.ops.kinetics.*`` custom
ops, and attention-layer objects shaped like the reference's benchmark layer
(``kinetics_amd.blocktopk_decoder``).  There is no CPU implementation.
"""
from . import ops  # noqa: F401  (registers torch.ops.kinetics.*)
from .blocktopk_decoder import BlockTopkPagedAttention, DensePagedAttention  # noqa: F401
from .decoder_layer import BlockTopkDecoderLayer, DenseDecoderLayer, GraphedLayer, qwen3_config  # noqa: F401

__all__ = ["ops", "BlockTopkPagedAttention", "DensePagedAttention", "BlockTopkDecoderLayer", "DenseDecoderLayer",
           "GraphedLayer", "qwen3_config"]
