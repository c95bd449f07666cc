"""lightning_attn import shim (linear_moe/sequence_modeling/lightning_attention/lightning_attention.py:6)."""
