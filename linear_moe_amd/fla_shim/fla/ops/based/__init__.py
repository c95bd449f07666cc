"""linear_moe/sequence_modeling/based/based.py:8; call ``parallel_based(q, k, v, True, True)`` (:72)."""
from linear_moe_amd.based import parallel_based

__all__ = ["parallel_based"]
