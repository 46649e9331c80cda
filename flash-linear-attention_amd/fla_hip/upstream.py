"""Backends that slot the HIP kernels into an unmodified upstream ``fla`` through its own plugin API
(``fla/ops/backends/__init__.py:33-220``; precedents ``fla/ops/gated_delta_rule/backends/flash_qla.py:32-132`` for a
whole operator and ``fla/modules/backends/triton_ascend`` for module functions).

    import fla_hip.upstream
    fla_hip.upstream.register()        # needs `fla` importable; registers for 'gated_delta_rule', 'modules' and 'kda'

Upstream's ``@dispatch`` then offers every call of ``chunk_gated_delta_rule``, ``causal_conv1d_fwd``,
``causal_conv1d_update_states``, ``causal_conv1d_update``, ``layer_norm_gated_fwd``, ``chunk_kda`` and ``fused_recurrent_kda_fwd``
(the KDA operator's token recurrence, ``fla/ops/kda/fused_recurrent.py:236``) to the verifier below first;
a rejected call (other device, a shape outside the kernels, gradients through an entry point that is forward only here) falls
through to upstream's own implementation.  The classes are built on whatever ``BaseBackend`` they are given, so the same code serves this
package's mirror of the registry (used by the tests)."""
from __future__ import annotations

import torch

ENV_VAR = 'FLA_HIP_GFX950'


def _on_gfx950(x) -> bool:
    return isinstance(x, torch.Tensor) and x.is_cuda and 'gfx950' in torch.cuda.get_device_properties(x.device).gcnArchName


def _needs_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


def make_backends(BaseBackend):
    """(operator backend, modules backend) as subclasses of the given ``BaseBackend``."""

    class HipGfx950Backend(BaseBackend):
        backend_type = 'hip_gfx950'
        package_name = 'fla_hip'
        env_var = ENV_VAR
        default_enable = True
        priority = 2                      # ahead of flash_qla (3) and the default

        def chunk_gated_delta_rule_verifier(self, q, k, v, g, beta, *args, cp_context=None, **kwargs):
            if not _on_gfx950(q):
                return False, 'not a gfx950 device'
            if cp_context is not None:
                return False, 'context parallelism is not supported'
            # (fp32 operands are left to upstream, which multiplies them as tf32: the chunk kernels here take 16-bit
            # operands and would round fp32 inputs to bf16 first - a silent loss of precision for such a caller)
            if q.dtype not in (torch.bfloat16, torch.float16):
                return False, f'dtype {q.dtype}'
            if k.shape[-1] > 256:
                return False, 'key head dim above 256'           # (upstream asserts the same: chunk_delta_h.py:712)
            return True, None

        def chunk_gated_delta_rule(self, *args, **kwargs):
            from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
            return chunk_gated_delta_rule(*args, **kwargs)

    class HipGfx950ModulesBackend(BaseBackend):
        backend_type = 'hip_gfx950'
        package_name = 'fla_hip'
        env_var = ENV_VAR
        default_enable = True
        priority = 2

        @staticmethod
        def _conv_ok(x, weight, *others):
            if not _on_gfx950(x):
                return False, 'not a gfx950 device'
            if _needs_grad(x, weight, *others):
                return False, 'forward only: a tensor requires grad'
            if x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
                return False, f'dtype {x.dtype}'
            return True, None

        def causal_conv1d_fwd_verifier(self, x, weight, bias=None, residual=None, initial_state=None, *args, **kwargs):
            if weight is None or weight.shape[-1] > 8:
                return False, 'kernel size above 8 (or no weight)'
            if kwargs.get('activation', args[1] if len(args) > 1 else None) not in (None, 'silu', 'swish'):
                return False, 'activation'
            return self._conv_ok(x, weight, bias, residual, initial_state)

        def causal_conv1d_fwd(self, *args, **kwargs):
            from fla_hip.modules import causal_conv1d_fwd
            return causal_conv1d_fwd(*args, **kwargs)

        def causal_conv1d_bwd_verifier(self, x, dy, dht, weight=None, *args, **kwargs):
            # (upstream calls this from its autograd function's backward, for a forward that may have run here)
            if weight is None or weight.shape[-1] > 8:
                return False, 'kernel size above 8 (or no weight)'
            if kwargs.get('activation') not in (None, 'silu', 'swish'):
                return False, 'activation'
            return self._conv_ok(x, weight)

        def causal_conv1d_bwd(self, *args, **kwargs):
            from fla_hip.modules import causal_conv1d_bwd
            return causal_conv1d_bwd(*args, **kwargs)

        def causal_conv1d_update_states_verifier(self, x, state_len, initial_state=None, cu_seqlens=None):
            if state_len > 8:
                return False, 'kernel size above 8'
            return self._conv_ok(x, None, initial_state)

        def causal_conv1d_update_states(self, *args, **kwargs):
            from fla_hip.modules import causal_conv1d_update_states
            return causal_conv1d_update_states(*args, **kwargs)

        def causal_conv1d_update_verifier(self, x, cache, residual=None, weight=None, bias=None, activation=None):
            if weight is None or weight.shape[-1] > 8 or cache is None or not cache.is_contiguous():
                return False, 'needs a weight of kernel size <= 8 and a contiguous cache'
            if activation not in (None, 'silu', 'swish'):
                return False, 'activation'
            return self._conv_ok(x, weight, bias, residual)

        def causal_conv1d_update(self, *args, **kwargs):
            from fla_hip.modules import causal_conv1d_update
            return causal_conv1d_update(*args, **kwargs)

        def layer_norm_gated_fwd_verifier(self, x, g, weight, bias, activation='swish', eps=1e-5, residual=None,
                                          out_dtype=None, residual_dtype=None, is_rms_norm=False):
            if not _on_gfx950(x):
                return False, 'not a gfx950 device'
            if _needs_grad(x, g, weight, bias, residual):
                return False, 'forward only: a tensor requires grad'
            if x.dtype not in (torch.bfloat16, torch.float16, torch.float32) or x.dim() != 2:
                return False, 'needs [T, D] rows of bf16, fp16 or fp32'
            if activation not in ('swish', 'silu', 'sigmoid'):
                return False, 'activation'
            return True, None

        def layer_norm_gated_fwd(self, *args, **kwargs):
            from fla_hip.modules import layer_norm_gated_fwd
            return layer_norm_gated_fwd(*args, **kwargs)

        def layer_norm_gated_bwd_verifier(self, dy, x, g, weight, bias, activation='swish', eps=1e-5, mean=None, rstd=None,
                                          dresidual=None, has_residual=False, is_rms_norm=False, x_dtype=None,
                                          recompute_output=False):
            if not _on_gfx950(x):
                return False, 'not a gfx950 device'
            if recompute_output:
                return False, 'recompute_output (the fused norm + linear layer)'
            if x.dtype not in (torch.bfloat16, torch.float16, torch.float32) or x.dim() != 2:
                return False, 'needs [T, D] rows of bf16, fp16 or fp32'
            if x.shape[1] > 2048:
                return False, 'feature dim above 2048'
            if activation not in ('swish', 'silu', 'sigmoid'):
                return False, 'activation'
            return True, None

        def layer_norm_gated_bwd(self, *args, **kwargs):
            from fla_hip.modules import layer_norm_gated_bwd
            return layer_norm_gated_bwd(*args, **kwargs)

    return HipGfx950Backend, HipGfx950ModulesBackend


def make_kda_backend(BaseBackend):
    """Backend for the 'kda' registry: the token recurrence (inference calls) and the chunked operator (forward and backward)."""

    class HipGfx950KDABackend(BaseBackend):
        backend_type = 'hip_gfx950'
        package_name = 'fla_hip'
        env_var = ENV_VAR
        default_enable = True
        priority = 2

        def fused_recurrent_kda_fwd_verifier(self, q, k, v, g, beta, A_log=None, dt_bias=None, initial_state=None, *args, **kwargs):
            if not _on_gfx950(q):
                return False, 'not a gfx950 device'
            if _needs_grad(q, k, v, g, beta, A_log, dt_bias, initial_state):
                return False, 'forward only: a tensor requires grad'
            if q.dtype not in (torch.bfloat16, torch.float16, torch.float32):
                return False, f'dtype {q.dtype}'
            if k.shape[-1] > 256:
                return False, 'key head dim above 256'
            if initial_state is not None and (initial_state.dtype != torch.float32 or not initial_state.is_contiguous()):
                return False, 'needs contiguous fp32 states'
            return True, None

        def fused_recurrent_kda_fwd(self, *args, **kwargs):
            from fla_hip.ops.kda import fused_recurrent_kda_fwd
            return fused_recurrent_kda_fwd(*args, **kwargs)

        def chunk_kda_verifier(self, q, k, v, g, beta, *args, cp_context=None, return_intermediate_states=False, **kwargs):
            if not _on_gfx950(q):
                return False, 'not a gfx950 device'
            if cp_context is not None:
                return False, 'context parallelism is not supported'
            # (calls that need gradients are taken too: chunk_kda here is differentiable in every input upstream's is)
            if q.dtype not in (torch.bfloat16, torch.float16):      # (fp32 operands: upstream's tf32 path, as above)
                return False, f'dtype {q.dtype}'
            if k.shape[-1] > 128:
                return False, 'key head dim above 128'
            return True, None

        def chunk_kda(self, *args, **kwargs):
            from fla_hip.ops.kda import chunk_kda
            return chunk_kda(*args, **kwargs)

    return HipGfx950KDABackend


def register() -> None:
    """Register the backends with upstream ``fla`` (ImportError when it is not installed).  Importing the two
    upstream packages first creates their registries (``gdr_registry``, ``modules_registry``, ``kda_registry``)."""
    import importlib
    backends = importlib.import_module('fla.ops.backends')
    gdr = importlib.import_module('fla.ops.gated_delta_rule.backends').gdr_registry
    modules = importlib.import_module('fla.modules.backends').modules_registry
    op_backend, modules_backend = make_backends(backends.BaseBackend)
    gdr.register(op_backend())
    modules.register(modules_backend())
    kda = importlib.import_module('fla.ops.kda.backends').kda_registry
    kda.register(make_kda_backend(backends.BaseBackend)())
