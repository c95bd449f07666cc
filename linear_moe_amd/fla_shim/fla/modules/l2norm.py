"""``l2_norm`` as linear_moe/sequence_modeling/linear_rnn.py:14 imports it: x * rsqrt(sum x^2 + eps)."""
from linear_moe_amd import l2_norm, l2_norm_fn  # noqa: F401

__all__ = ["l2_norm", "l2_norm_fn"]
