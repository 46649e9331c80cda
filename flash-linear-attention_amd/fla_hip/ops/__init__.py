from fla_hip.ops.comba import chunk_comba, fused_recurrent_comba
from fla_hip.ops.delta_rule import chunk_delta_rule, fused_recurrent_delta_rule
from fla_hip.ops.kda import chunk_kda, fused_recurrent_kda
from fla_hip.ops.gated_delta_rule import (
    chunk_gated_delta_rule,
    chunk_gdn,
    fused_recurrent_gated_delta_rule,
    fused_recurrent_gdn,
)

__all__ = ['chunk_delta_rule', 'fused_recurrent_delta_rule', 'chunk_gated_delta_rule', 'chunk_gdn', 'fused_recurrent_gated_delta_rule', 'fused_recurrent_gdn',
           'chunk_kda', 'fused_recurrent_kda', 'chunk_comba', 'fused_recurrent_comba']
