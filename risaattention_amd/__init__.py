"""MI355X (gfx950) implementation of RISA's quantized attention path.

The public names and signatures are those of the reference package
``risa_attention`` (src/risa_attention/__init__.py:17-31), so
``import risaattention_amd as risa_attention`` is a drop-in for this path.
"""

from .attend import int8_attention_from_prequantized
from .dense import int8_attention
from .fp32_patterns import build_retained_mass_pattern, measure_pattern_recall
from .native import is_available as int8_attention_is_available
from .patterns import (
    construct_sparse_int8_attention,
    construct_sparse_int8_attention_from_prequantized,
    sparse_int8_attention,
)
from .permutation import KVPermutation, prepare_kv_permutation
from .prepare import prequantize_int8_attention
from .types import PrequantizedInt8Attention, RetainedMassPattern

__all__ = [
    "KVPermutation",
    "prepare_kv_permutation",
    "PrequantizedInt8Attention",
    "RetainedMassPattern",
    "build_retained_mass_pattern",
    "construct_sparse_int8_attention",
    "construct_sparse_int8_attention_from_prequantized",
    "int8_attention",
    "int8_attention_from_prequantized",
    "int8_attention_is_available",
    "measure_pattern_recall",
    "prequantize_int8_attention",
    "sparse_int8_attention",
]

__version__ = "0.2.0+gfx950"
