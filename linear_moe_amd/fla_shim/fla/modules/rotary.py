"""``RotaryEmbedding`` as linear_moe/model/common_modules/__init__.py:5 imports it.  The name has to resolve for the
reference's token mixers to import at all (each of them imports that package); the linear-attention layers never
apply a rotary embedding (``rotary_pos_emb = None``, linear_moe/sequence_modeling/linear_attention.py:185), so
this library has no kernel for it and says so when the class is used."""
import torch


class RotaryEmbedding(torch.nn.Module):
    def __init__(self, *args, **kwargs):
        super().__init__()
        raise NotImplementedError(
            "fla.modules.rotary.RotaryEmbedding: rotary embeddings are not on the linear-attention path and are "
            "not provided by linear_moe_amd")


__all__ = ["RotaryEmbedding"]
