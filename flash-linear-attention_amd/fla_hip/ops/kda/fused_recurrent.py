"""``fused_recurrent_kda``: the token recurrence of the KDA operator (the gated delta rule with a decay per key
feature), forward only, with the signatures of fla/ops/kda/fused_recurrent.py:236-260 (``fused_recurrent_kda_fwd``, the
serving form with state pools) and :341-492 (``fused_recurrent_kda``).  Both run the token-recurrence kernel of the gated
delta rule through ``gdn_fused_recurrent_kda_fwd``; the chunked prefill is ``chunk_kda`` (chunk.py)."""
from __future__ import annotations

import warnings

import torch

from fla_hip.ops.gated_delta_rule.fused_recurrent import fused_recurrent_gated_delta_rule_fwd


def fused_recurrent_kda_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    A_log: torch.Tensor | None = None,
    dt_bias: torch.Tensor | None = None,
    initial_state: torch.Tensor | None = None,
    scale: float | None = None,
    output_final_state: bool = False,
    inplace_final_state: bool = True,
    state_v_first: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
    ssm_state_indices: torch.Tensor | None = None,
    num_accepted_tokens: torch.Tensor | None = None,
    use_qk_l2norm_in_kernel: bool = False,
    use_gate_in_kernel: bool = False,
    use_beta_sigmoid_in_kernel: bool = False,
    allow_neg_eigval: bool = False,
    lower_bound: float | None = None,
    out: torch.Tensor | None = None,
    **kwargs,
) -> tuple[torch.Tensor, torch.Tensor]:
    """g ``[B, T, HV, K]``: log decays, or the raw gate input with ``use_gate_in_kernel`` (then
    ``-exp(A_log) * softplus(g + dt_bias)``, or ``lower_bound * sigmoid(exp(A_log) * (g + dt_bias))`` when a lower bound is
    given; ``A_log [HV]``, ``dt_bias [HV * K]``).  ``inplace_final_state`` (the default here, as in the reference)
    writes the final state over ``initial_state``; with ``ssm_state_indices`` that tensor is a pool of slots."""
    if scale is None:
        scale = k.shape[-1] ** -0.5
    if inplace_final_state and initial_state is None:
        raise ValueError('`inplace_final_state=True` requires `initial_state`.')
    if use_gate_in_kernel:
        gate_mode = 2 if lower_bound is not None else 1
        if dt_bias is not None and dt_bias.numel() != v.shape[2] * k.shape[-1]:
            raise ValueError(f'dt_bias must have HV * K = {v.shape[2] * k.shape[-1]} elements, got {dt_bias.numel()}')
    else:
        gate_mode, A_log, dt_bias = 0, None, None
    o, final_state = fused_recurrent_gated_delta_rule_fwd(
        q, k, v, None, g, None, beta, A_log, dt_bias, scale, initial_state, output_final_state,
        use_qk_l2norm_in_kernel, use_beta_sigmoid_in_kernel, allow_neg_eigval, state_v_first, cu_seqlens,
        inplace_final_state, ssm_state_indices, num_accepted_tokens,
        kda_gate_mode=gate_mode, lower_bound=0.0 if lower_bound is None else lower_bound)
    if out is not None:
        if out.shape != v.shape:
            raise ValueError(f'out must have the shape of v {tuple(v.shape)}, got {tuple(out.shape)}')
        out.copy_(o)
        o = out
    return o, final_state


@torch.compiler.disable
def fused_recurrent_kda(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    A_log: torch.Tensor | None = None,
    dt_bias: torch.Tensor | None = None,
    scale: float | None = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    use_gate_in_kernel: bool = False,
    use_beta_sigmoid_in_kernel: bool = False,
    allow_neg_eigval: bool = False,
    lower_bound: float | None = None,
    state_v_first: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
    **kwargs,
) -> tuple[torch.Tensor, torch.Tensor]:
    r"""q, k ``[B, T, H, K]``; v ``[B, T, HV, V]`` (``HV % H == 0``); g ``[B, T, HV, K]``; beta ``[B, T, HV]``.
    Returns ``(o [B, T, HV, V], final_state [N, HV, K, V] fp32 or None)``; the initial state is never written."""
    if 'transpose_state_layout' in kwargs:
        if state_v_first:
            raise ValueError('Cannot pass both `state_v_first` and the deprecated `transpose_state_layout`.')
        warnings.warn('`transpose_state_layout` is deprecated and renamed to `state_v_first`.',
                      DeprecationWarning, stacklevel=2)
        state_v_first = kwargs.pop('transpose_state_layout')
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
    if allow_neg_eigval and not use_beta_sigmoid_in_kernel:
        raise ValueError('`allow_neg_eigval=True` requires `use_beta_sigmoid_in_kernel=True`.')
    return fused_recurrent_kda_fwd(
        q=q, k=k, v=v, g=g, beta=beta, A_log=A_log, dt_bias=dt_bias, scale=scale, initial_state=initial_state,
        inplace_final_state=False, output_final_state=output_final_state,
        use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, use_gate_in_kernel=use_gate_in_kernel,
        use_beta_sigmoid_in_kernel=use_beta_sigmoid_in_kernel, allow_neg_eigval=allow_neg_eigval,
        lower_bound=lower_bound, cu_seqlens=cu_seqlens, state_v_first=state_v_first)
