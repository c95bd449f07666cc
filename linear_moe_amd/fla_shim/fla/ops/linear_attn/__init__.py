"""linear_moe/sequence_modeling/basic_linear_attention/basic_linear_attention.py:11-12 (also based.py:9,
rebased.py:9); call ``impl(q, k, v, normalize=...)``."""
from linear_moe_amd import chunk_linear_attn

fused_chunk_linear_attn = chunk_linear_attn
fused_recurrent_linear_attn = chunk_linear_attn

__all__ = ["chunk_linear_attn", "fused_chunk_linear_attn", "fused_recurrent_linear_attn"]
