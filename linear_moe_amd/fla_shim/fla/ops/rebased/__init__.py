"""linear_moe/sequence_modeling/rebased/rebased.py:9; call ``parallel_rebased(q, k, v, eps, True, True)`` (:79)."""
from linear_moe_amd.based import parallel_rebased

__all__ = ["parallel_rebased"]
