"""The caller of the gated delta rule path: the Gated DeltaNet token-mixing layer (inference only)."""
from fla_hip.layers.gated_deltanet import GatedDeltaNet, LayerCache

__all__ = ['GatedDeltaNet', 'LayerCache']
