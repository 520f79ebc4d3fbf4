"""Constants of the nested E8 codec shared by containers and kernels.

Mirrors the identifiers of nestquant/core/codec.py:15-17 so records written by either
implementation name the same semantics.
"""

UPSTREAM_CODEC_SEMANTICS = "e8_upstream_half_coset_tie_v1"
LEGACY_CODEC_SEMANTICS = "e8_legacy_integer_coset_tie_v1"
CURRENT_CODEC_SEMANTICS = UPSTREAM_CODEC_SEMANTICS
STATELESS_DITHER_ALGORITHM = "lcg31_mix_v1"
STATELESS_MODULUS = 1 << 31
E8_DIMENSION = 8
