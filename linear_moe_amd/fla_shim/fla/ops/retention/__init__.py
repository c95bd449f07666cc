"""linear_moe/sequence_modeling/retention/retention.py:11-12; call ``impl(q, k, v)``."""
from linear_moe_amd import chunk_retention

fused_chunk_retention = chunk_retention
fused_recurrent_retention = chunk_retention
parallel_retention = chunk_retention

__all__ = ["chunk_retention", "fused_chunk_retention", "fused_recurrent_retention", "parallel_retention"]
