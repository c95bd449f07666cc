"""linear_moe/sequence_modeling/gla/gla.py:11 and hgrn2/hgrn2.py:11 import these three names and call
whichever ``la_mode`` selects as ``impl(q, k, v, gk)``."""
from linear_moe_amd import chunk_gla, fused_recurrent_gla

fused_chunk_gla = chunk_gla

__all__ = ["chunk_gla", "fused_chunk_gla", "fused_recurrent_gla"]
