"""The two memory-bound steps either side of the gated delta rule in the layer
(fla/layers/gated_deltanet.py:246-300, :355-359): the causal short convolution in front of it and the
gated normalisation behind it, with the reference's names (fla/modules/__init__.py)."""
from fla_hip.modules.convolution import (
    ShortConvolution,
    causal_conv1d,
    causal_conv1d_bwd,
    causal_conv1d_fwd,
    causal_conv1d_update,
    causal_conv1d_update_states,
)
from fla_hip.modules.fused_norm_gate import (
    FusedLayerNormGated,
    FusedLayerNormSwishGate,
    FusedRMSNormGated,
    FusedRMSNormSwishGate,
    layer_norm_gated,
    layer_norm_gated_bwd,
    layer_norm_gated_fwd,
    rms_norm_gated,
)

__all__ = [
    'ShortConvolution', 'causal_conv1d', 'causal_conv1d_fwd', 'causal_conv1d_bwd', 'causal_conv1d_update', 'causal_conv1d_update_states',
    'FusedLayerNormGated', 'FusedLayerNormSwishGate', 'FusedRMSNormGated', 'FusedRMSNormSwishGate',
    'layer_norm_gated', 'layer_norm_gated_fwd', 'layer_norm_gated_bwd', 'rms_norm_gated',
]
