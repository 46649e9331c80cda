from .chunk import chunk_kda, chunk_kda_fwd
from .fused_recurrent import fused_recurrent_kda, fused_recurrent_kda_fwd

__all__ = ['chunk_kda', 'chunk_kda_fwd', 'fused_recurrent_kda', 'fused_recurrent_kda_fwd']
