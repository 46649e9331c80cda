from .fused_recurrent import fused_recurrent_kda, fused_recurrent_kda_fwd

__all__ = ['fused_recurrent_kda', 'fused_recurrent_kda_fwd']
