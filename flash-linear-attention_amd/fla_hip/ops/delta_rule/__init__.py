from .chunk import chunk_delta_rule
from .fused_chunk import fused_chunk_delta_rule
from .fused_recurrent import fused_recurrent_delta_rule

__all__ = ['chunk_delta_rule', 'fused_chunk_delta_rule', 'fused_recurrent_delta_rule']
