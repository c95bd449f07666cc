"""linear_moe/sequence_modeling/gated_deltanet/gated_deltanet.py:11; call at :112
``impl(q, k, v, gk, beta, head_first=False)``."""
from linear_moe_amd import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule

__all__ = ["chunk_gated_delta_rule", "fused_recurrent_gated_delta_rule"]
