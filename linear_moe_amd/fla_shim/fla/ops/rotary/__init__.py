"""``apply_rotary`` as linear_moe/model/common_modules/rotary.py:10 imports it (used at :53 and :86 by the softmax
layers' rotary autograd function, never by the linear-attention layers): resolves, raises when called."""


def apply_rotary(*args, **kwargs):
    raise NotImplementedError(
        "fla.ops.rotary.apply_rotary: rotary embeddings are not on the linear-attention path and are not provided "
        "by linear_moe_amd")


__all__ = ["apply_rotary"]
