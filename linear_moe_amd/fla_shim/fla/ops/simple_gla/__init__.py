from linear_moe_amd import chunk_simple_gla, fused_recurrent_simple_gla  # noqa: F401

__all__ = ["chunk_simple_gla", "fused_recurrent_simple_gla"]
