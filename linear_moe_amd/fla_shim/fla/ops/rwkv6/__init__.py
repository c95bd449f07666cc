"""linear_moe/sequence_modeling/rwkv6/rwkv6.py:11 imports these names; the RWKV-6 recurrence is a different
operator family from the three chunk ops this library builds: the names resolve and raise when called."""


def _unsupported(name):
    def fn(*args, **kwargs):
        raise NotImplementedError(f"fla.ops.rwkv6.{name}: the RWKV-6 recurrence is not provided by linear_moe_amd")
    fn.__name__ = name
    return fn


chunk_rwkv6 = _unsupported("chunk_rwkv6")
fused_recurrent_rwkv6 = _unsupported("fused_recurrent_rwkv6")

__all__ = ["chunk_rwkv6", "fused_recurrent_rwkv6"]
