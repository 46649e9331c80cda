from .chunk import chunk_gated_delta_rule, chunk_gdn
from .fused_recurrent import fused_recurrent_gated_delta_rule, fused_recurrent_gdn
from .naive import naive_chunk_gated_delta_rule, naive_recurrent_gated_delta_rule

__all__ = [
    'chunk_gated_delta_rule', 'chunk_gdn',
    'fused_recurrent_gated_delta_rule', 'fused_recurrent_gdn',
    'naive_chunk_gated_delta_rule',
    'naive_recurrent_gated_delta_rule',
]
