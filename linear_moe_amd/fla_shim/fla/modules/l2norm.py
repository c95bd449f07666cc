"""``l2_norm`` as linear_moe/sequence_modeling/linear_rnn.py:14 imports it: x * rsqrt(sum x^2 + eps)."""
from linear_moe_amd.gated_delta_rule import _l2norm as l2_norm  # noqa: F401

__all__ = ["l2_norm"]
