"""Operator entry points, same names as the reference package
palimpsa/ops/palimpsa/__init__.py:4-5."""
from .chunk import ChunkPalimpsa, chunk_palimpsa
from .fused_recurrent import FusedRecurrentPalimpsaFunction, fused_recurrent_palimpsa
from .naive import palimpsa_ref
from .decode import DecodeStep, mu_from_cache, mu_to_cache

__all__ = [
    "chunk_palimpsa",
    "fused_recurrent_palimpsa",
    "palimpsa_ref",
    "ChunkPalimpsa",
    "FusedRecurrentPalimpsaFunction",
    "DecodeStep",
    "mu_to_cache",
    "mu_from_cache",
]
