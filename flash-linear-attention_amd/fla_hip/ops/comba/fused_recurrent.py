"""``fused_recurrent_comba`` with the signature of fla/ops/comba/fused_recurrent.py:225-335 (mind the order: q, k, p, v).
The token recurrence (predict with p on the undecayed state, decay, write k; fused_recurrent.py:85-105) is the map the
chunked kernels compute, so the call runs on them; there is no separate token-by-token kernel for this operator.
The reference's recurrent kernel computes in fp32 whatever the inputs' dtype; here fp32 inputs are handed to the kernels
as fp16 operands (11 significant bits; values beyond 65504 overflow), which keeps the result within the reference's
0.002 bar for this entry point (tests/ops/test_comba.py:117-118)."""
from __future__ import annotations

import torch

from fla_hip.ops.gated_delta_rule._common import forward_only

from .chunk import check_comba_args, chunk_comba_fwd


@torch.compiler.disable
def fused_recurrent_comba(
    q: torch.Tensor,
    k: torch.Tensor,
    p: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor = None,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
):
    r"""Args as ``chunk_comba`` (``v``: ``[B, T, HV, V]``, grouped value heads allowed), in the reference's order
    ``q, k, p, v, g, beta``.  A beta per value column (``[B, T, HV, V]``) is not covered.

    Returns:
        ``(o [B, T, HV, V] in q's dtype, final_state [N, HV, K, V] fp32 or None)``.
    """
    if p is None:
        p = k
    if beta is None:
        beta = torch.ones_like(g)
    if beta.dim() == 4:
        raise NotImplementedError('fused_recurrent_comba: a beta per value column is outside this build')
    check_comba_args(q, k, v, p, g, beta, initial_state, cu_seqlens)
    forward_only('fused_recurrent_comba', q, k, p, v, g, beta, initial_state)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    return chunk_comba_fwd(q, k, v, p, g, beta, scale, initial_state, output_final_state, use_qk_l2norm_in_kernel, cu_seqlens,
                           fp32_as=torch.float16)
