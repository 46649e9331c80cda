"""``fused_recurrent_delta_rule``: the token recurrence of the delta rule without gates, forward only, with
the signature of fla/ops/delta_rule/fused_recurrent.py:443-532; the gated kernel with g absent."""
from __future__ import annotations

import torch

from fla_hip.ops.gated_delta_rule.fused_recurrent import fused_recurrent_gated_delta_rule_fwd


@torch.compiler.disable
def fused_recurrent_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor = None,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    r"""q, k ``[B, T, H, K]``, v ``[B, T, H, V]``, beta ``[B, T, H]`` or ``[B, T, H, V]`` (ones when omitted).
    Returns ``(o, final_state [N, H, K, V] fp32 or None)``."""
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f'The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`.'
                f'Please flatten variable-length inputs before processing.')
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(
                f'The number of initial states is expected to be equal to the number of input sequences, '
                f'i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.')
    if scale is None:
        scale = k.shape[-1] ** -0.5
    else:
        assert scale > 0, 'scale must be positive'
    return fused_recurrent_gated_delta_rule_fwd(
        q, k, v, beta=beta, scale=scale, initial_state=initial_state, output_final_state=output_final_state,
        use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, cu_seqlens=cu_seqlens)
