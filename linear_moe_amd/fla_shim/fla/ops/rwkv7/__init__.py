"""linear_moe/sequence_modeling/rwkv7/rwkv7.py:11 imports these names; the RWKV-7 recurrence is a different
operator family from the three chunk ops this library builds: the names resolve and raise when called."""


def _unsupported(name):
    def fn(*args, **kwargs):
        raise NotImplementedError(f"fla.ops.rwkv7.{name}: the RWKV-7 recurrence is not provided by linear_moe_amd")
    fn.__name__ = name
    return fn


chunk_rwkv7 = _unsupported("chunk_rwkv7")
fused_recurrent_rwkv7 = _unsupported("fused_recurrent_rwkv7")

__all__ = ["chunk_rwkv7", "fused_recurrent_rwkv7"]
