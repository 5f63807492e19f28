"""
MI355X (gfx950) implementation of torch-harmonics' spherical neighborhood attention:
the NeighborhoodAttentionS2 module, its autograd op and the layout conversions, over
hand-written HIP kernels in libs2attn.so.
"""

from . import _lib
from ._layout import to_nchw, to_nhwc
from .attention import NeighborhoodAttentionS2
from .neighborhood import precompute_neighborhood_s2
from .ops import _neighborhood_s2_attention_optimized, neighborhood_s2_attention
from .quadrature import precompute_latitudes, precompute_longitudes

__all__ = [
    "NeighborhoodAttentionS2",
    "_neighborhood_s2_attention_optimized",
    "neighborhood_s2_attention",
    "to_nhwc",
    "to_nchw",
    "precompute_neighborhood_s2",
    "precompute_latitudes",
    "precompute_longitudes",
    "optimized_kernels_is_available",
]


def optimized_kernels_is_available() -> bool:
    """True when libs2attn.so has been built (attention_helpers.cpp:43-54 answers the same question for the reference)."""
    return _lib.is_built()
