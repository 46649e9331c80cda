"""Backends of the 'gated_delta_rule' operation.  None is registered by default: the
decorated functions in this package already are the HIP implementation.  The registry
exists so that callers can slot in their own ``BaseBackend`` exactly as with the reference
(fla/ops/gated_delta_rule/backends/__init__.py:1-20)."""
from fla_hip.ops.backends import BackendRegistry

gated_delta_rule_registry = BackendRegistry('gated_delta_rule')

__all__ = ['gated_delta_rule_registry']
