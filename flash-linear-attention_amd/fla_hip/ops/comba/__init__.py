from .chunk import chunk_comba, chunk_comba_fwd
from .fused_recurrent import fused_recurrent_comba

__all__ = ['chunk_comba', 'chunk_comba_fwd', 'fused_recurrent_comba']
