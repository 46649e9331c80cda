"""fla_hip - drop-in for ``fla.ops.gated_delta_rule`` on AMD MI355X (gfx950).

Public surface mirrors the reference for this one path:
``fla_hip.ops.gated_delta_rule.{chunk_gated_delta_rule, fused_recurrent_gated_delta_rule,
chunk_gdn, fused_recurrent_gdn, naive_*}``; ``fla_hip.ops.backends`` (dispatch / registry);
``fla_hip.utils`` (input_guard, tensor_cache, assert_close).  Compute is done only by the
HIP library ``_C/libgdn_hip.so`` through its C ABI; there is no CPU or eager fallback.
"""
from fla_hip.ops.gated_delta_rule import (
    chunk_gated_delta_rule,
    chunk_gdn,
    fused_recurrent_gated_delta_rule,
    fused_recurrent_gdn,
    naive_chunk_gated_delta_rule,
    naive_recurrent_gated_delta_rule,
)

__version__ = '0.1.0'

__all__ = [
    'chunk_gated_delta_rule', 'chunk_gdn',
    'fused_recurrent_gated_delta_rule', 'fused_recurrent_gdn',
    'naive_chunk_gated_delta_rule', 'naive_recurrent_gated_delta_rule',
]
