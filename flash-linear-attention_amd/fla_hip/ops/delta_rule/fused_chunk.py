"""``fused_chunk_delta_rule``: the name the reference still exports (fla/ops/delta_rule/fused_chunk.py:8-11) for an entry
point it has retired; calling it raises, there as here."""


def fused_chunk_delta_rule(**kwargs):
    raise NotImplementedError('fused_chunk_delta_rule is deprecated. Please use chunk_delta_rule instead.')
