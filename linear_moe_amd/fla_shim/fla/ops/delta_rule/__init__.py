"""linear_moe/sequence_modeling/deltanet/deltanet.py:11-12; calls at :125-130
``impl(q, k, v, beta)`` (fused_recurrent) or ``impl(q, k, v, beta, chunk_size)``."""
from linear_moe_amd import chunk_delta_rule, fused_recurrent_delta_rule

fused_chunk_delta_rule = chunk_delta_rule

__all__ = ["chunk_delta_rule", "fused_chunk_delta_rule", "fused_recurrent_delta_rule"]
