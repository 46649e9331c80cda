from .chunk import chunk_comba, chunk_comba_fwd
from .fused_recurrent import fused_recurrent_comba
from .naive import naive_chunk_comba, naive_recurrent_comba

__all__ = ['chunk_comba', 'chunk_comba_fwd', 'fused_recurrent_comba', 'naive_chunk_comba', 'naive_recurrent_comba']
