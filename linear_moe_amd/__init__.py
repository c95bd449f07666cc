"""MI355X-native chunked linear-attention ops behind flash-linear-attention's call signatures.

Drop-in for the ``fla.ops`` callables the reference's token mixers import
(``linear_moe/sequence_modeling/{gla,retention,gated_deltanet,deltanet,basic_linear_attention}``).
All compute runs in hand-written HIP kernels (``csrc/``) reached through the C ABI of
``liblmoe_hip.so`` (``include/lmoe.h``); there is no fallback path.
"""
from ._host import forget_cu_seqlens, prepare_cu_seqlens  # noqa: F401
from .delta_rule import chunk_delta_rule  # noqa: F401
from .gated_delta_rule import chunk_gated_delta_rule  # noqa: F401
from . import lasp  # noqa: F401
from .feature_map import KeyBlocks, quad_feature_map, rebased_feature_map, taylor_feature_map  # noqa: F401
from .gates import gdn_gates, gla_gate, hgrn2_gates  # noqa: F401
from .gla import chunk_gla  # noqa: F401
from .layer_io import gdn_mixer_core, gdn_qkv_prologue, swish_gate_relayout  # noqa: F401
from .l2norm import l2_norm, l2_norm_fn, silu_l2_norm  # noqa: F401
from .rmsnorm import RMSNorm, rms_norm_fn, rms_norm_swish_gate  # noqa: F401
from .lightning import lightning_attn2, lightning_attn2_no_decay  # noqa: F401
from .linear_attn import chunk_linear_attn  # noqa: F401
from .mom import MomPlan, mom_combine, mom_pack, mom_plan  # noqa: F401
from .recurrent import (fused_recurrent_delta_rule, fused_recurrent_gated_delta_rule, fused_recurrent_gla,  # noqa: F401
                        fused_recurrent_simple_gla)
from .retention import chunk_retention  # noqa: F401
from .simple_gla import chunk_simple_gla  # noqa: F401

__all__ = ["chunk_simple_gla", "chunk_gla", "chunk_gated_delta_rule", "chunk_delta_rule", "chunk_retention", "chunk_linear_attn",
           "lightning_attn2", "lightning_attn2_no_decay", "l2_norm", "l2_norm_fn", "silu_l2_norm", "gdn_qkv_prologue", "gdn_mixer_core", "swish_gate_relayout", "rms_norm_fn",
           "rms_norm_swish_gate", "RMSNorm", "gdn_gates", "gla_gate", "fused_recurrent_simple_gla", "fused_recurrent_gla",
           "fused_recurrent_gated_delta_rule", "fused_recurrent_delta_rule", "mom_plan", "mom_pack", "mom_combine", "MomPlan",
           "prepare_cu_seqlens", "forget_cu_seqlens", "hgrn2_gates", "taylor_feature_map", "rebased_feature_map", "quad_feature_map", "KeyBlocks", "lasp"]
