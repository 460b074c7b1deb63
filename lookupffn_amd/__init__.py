"""lookupffn_amd: the LookupFFN layer of mlpen/LookupFFN on hand-written gfx950
(MI355X) kernels, behind the reference's own module and operator names.

The kernels live in liblookupffn_hip.so (C ABI: include/lookupffn_hip.h), built
by ``python -m lookupffn_amd._build``.  There is no CPU or PyTorch fallback.
"""
from . import _lib  # noqa: F401
from .bh4 import (FastHadamardTransform, FastHadamardTransformDim512, FastHadamardTransformDim1024, bh4,
                  bh4_cuda, fast_hadamard_transform, hadamard, hadamard_transform)
from .compute_code_score import ComputeCodeScore, bin2dec, compute_code_score, compute_code_score_torch
from .gather import (LookupGather, WeightedVectorGatherAdd, gather, indexed_inner_product, lookup_gather,
                     weighted_gather_add, weighted_vector_gather_add, weighted_vector_scatter_add)
from .lookup import BH4, Hashing, LookupFFN
from .encoder import Attention, Encoder, EncoderLayer, Lookup, RobertaEmbeddings

__all__ = [
    "BH4", "Hashing", "LookupFFN",
    "Attention", "EncoderLayer", "Encoder", "Lookup", "RobertaEmbeddings",
    "bh4", "bh4_cuda", "hadamard", "hadamard_transform", "fast_hadamard_transform",
    "FastHadamardTransform", "FastHadamardTransformDim512", "FastHadamardTransformDim1024",
    "compute_code_score", "compute_code_score_torch", "bin2dec", "ComputeCodeScore",
    "gather", "weighted_gather_add", "weighted_vector_gather_add", "indexed_inner_product",
    "weighted_vector_scatter_add", "WeightedVectorGatherAdd", "LookupGather", "lookup_gather",
]
