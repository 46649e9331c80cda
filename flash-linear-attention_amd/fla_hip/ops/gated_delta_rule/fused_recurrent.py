"""``fused_recurrent_gated_delta_rule``: same signature, defaults, validation and error
types as fla/ops/gated_delta_rule/fused_recurrent.py:309-475; the single Triton launch
(:184-250) is replaced by one call into libgdn_hip.so (``gdn_fused_recurrent_fwd``)."""
from __future__ import annotations

import warnings

import torch

from fla_hip import _lib
from fla_hip.ops.gated_delta_rule._common import (
    check_operand_shapes,
    aligned16,
    as_f32,
    current_stream_ptr,
    dtype_code,
    ptr,
    require_gpu,
    unify_gate_beta,
    unify_qkv,
)
from fla_hip.ops.utils.index import max_seq_len
from fla_hip.utils import input_guard


@input_guard
def fused_recurrent_gated_delta_rule_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor | None = None,
    gk: torch.Tensor | None = None,
    gv: torch.Tensor | None = None,
    beta: torch.Tensor | None = None,
    A_log: torch.Tensor | None = None,
    dt_bias: torch.Tensor | None = None,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    use_beta_sigmoid_in_kernel: bool = False,
    allow_neg_eigval: bool = False,
    state_v_first: bool = False,
    cu_seqlens: torch.Tensor | None = None,
    inplace_final_state: bool = False,
    ssm_state_indices: torch.Tensor | None = None,
    num_accepted_tokens: torch.Tensor | None = None,
    kda_gate_mode: int | None = None,
    lower_bound: float = 0.0,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Allocates ``o`` (v's dtype) and the fp32 final state, then launches the HIP kernel on
    the current stream.  With ``inplace_final_state`` the final state is written over
    ``initial_state`` (which must then be fp32, or bf16 for states kept in bf16, and contiguous) and that tensor is returned.
    With ``ssm_state_indices`` the states are slots of the pool ``initial_state
    [num_slots, HV, K, V]``: ``[N]`` names one slot per sequence, updated in place; ``[N, T]`` names
    a slot per token (the state after token t goes to slot ``[n, t]``, and the sequence starts from
    slot ``[n, num_accepted_tokens[n] - 1]``, or ``[n, 0]``).  Without ``inplace_final_state`` the
    pool is only read and the states after every token are returned as ``[B * T, HV, K, V]``.
    ``kda_gate_mode`` (0, 1, 2) selects the KDA operator's entry point: ``gk`` is then its per-key gate ``g``
    (mode 0: log decays; 1, 2: raw, activated in the kernel with ``A_log [HV]``, ``dt_bias [HV, K]`` and
    ``lower_bound``), and ``g``, ``gv`` must be absent."""
    dev = require_gpu(q, k, v)
    check_operand_shapes(q, k, v, g=g, beta=beta, gk=gk, gv=gv, beta_per_column=True)
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    q, k, v = unify_qkv(q, k, v)
    g, beta, gb_code = unify_gate_beta(g, beta)
    gk, gv, A_log, dt_bias = as_f32(gk), as_f32(gv), as_f32(A_log), as_f32(dt_bias)
    if A_log is not None and A_log.numel() != HV:
        raise ValueError(f'A_log must have {HV} entries, got {A_log.numel()}')
    if dt_bias is not None and dt_bias.numel() != (HV * K if kda_gate_mode is not None else HV):
        raise ValueError(f'dt_bias must have {HV * K if kda_gate_mode is not None else HV} entries, got {dt_bias.numel()}')

    # The kernel moves 16-byte pieces of state rows.  Head dims that are not multiples of 4 are zero-padded
    # here (zero key features and zero value columns change nothing else) and the results cut back.
    KP, VP = (K + 3) // 4 * 4, (V + 3) // 4 * 4
    padded = (KP, VP) != (K, V)
    if padded:
        if inplace_final_state or ssm_state_indices is not None:
            raise NotImplementedError('in-place and pooled states need head dims that are multiples of 4')
        pad = torch.nn.functional.pad
        q, k, v = pad(q, (0, KP - K)), pad(k, (0, KP - K)), pad(v, (0, VP - V))
        gk = None if gk is None else pad(gk, (0, KP - K))
        if kda_gate_mode and dt_bias is not None:
            dt_bias = pad(dt_bias.reshape(HV, K), (0, KP - K))
        gv = None if gv is None else pad(gv, (0, VP - V))
        if beta is not None and beta.ndim == v.ndim:
            beta = pad(beta, (0, VP - V))
        if initial_state is not None:
            initial_state = pad(initial_state, (0, KP - K, 0, VP - V) if state_v_first else (0, VP - V, 0, KP - K))

    flags = 0
    if use_qk_l2norm_in_kernel:
        flags |= _lib.FLAG_QK_L2NORM
    if use_beta_sigmoid_in_kernel:
        flags |= _lib.FLAG_BETA_SIGMOID
    if allow_neg_eigval:
        flags |= _lib.FLAG_NEG_EIGVAL
    if state_v_first:
        flags |= _lib.FLAG_STATE_V_FIRST
    if beta is not None and beta.ndim == v.ndim:
        flags |= _lib.FLAG_BETA_VECTOR
    if cu_seqlens is not None:
        if cu_seqlens.dtype == torch.int32:
            flags |= _lib.FLAG_CU_INT32
        elif cu_seqlens.dtype != torch.int64:
            cu_seqlens = cu_seqlens.long()
        if cu_seqlens.device != dev:
            cu_seqlens = cu_seqlens.to(dev)

    state_shape = (N, HV, VP, KP) if state_v_first else (N, HV, KP, VP)
    h0 = initial_state
    slots = accepted = None
    slots_stride = 1
    per_token_out = False
    if num_accepted_tokens is not None and (ssm_state_indices is None or ssm_state_indices.ndim != 2):
        raise ValueError('num_accepted_tokens needs ssm_state_indices of shape (N, T)')
    if ssm_state_indices is not None:
        if h0 is None:
            raise ValueError('ssm_state_indices needs the state pool as initial_state')
        if ssm_state_indices.ndim == 1:
            if not inplace_final_state:
                raise ValueError('ssm_state_indices of shape (N,) needs inplace_final_state=True')
            if ssm_state_indices.shape[0] != N:
                raise ValueError(f'ssm_state_indices must have shape ({N},), got {tuple(ssm_state_indices.shape)}')
        elif ssm_state_indices.ndim == 2:
            if ssm_state_indices.shape[0] != N:
                raise ValueError(f'ssm_state_indices must have {N} rows, got {tuple(ssm_state_indices.shape)}')
            # a slot per token: the kernel reads row n at column t for every token t of sequence n (packed input: the
            # longest sequence decides, from the host copy of the boundaries, memoised per cu_seqlens tensor)
            longest = T if cu_seqlens is None else max_seq_len(cu_seqlens)
            if ssm_state_indices.shape[1] < longest:
                raise ValueError(f'ssm_state_indices needs a slot for each of the {longest} tokens of a sequence, '
                                 f'got {tuple(ssm_state_indices.shape)}')
            if inplace_final_state:
                flags |= _lib.FLAG_SLOT_PER_TOKEN
            slots_stride = ssm_state_indices.shape[1]
        else:
            raise ValueError('ssm_state_indices must have one or two dimensions')
        slots = ssm_state_indices.to(dev)
        if slots.dtype == torch.int32:
            flags |= _lib.FLAG_SLOT_INT32
        elif slots.dtype != torch.int64:
            slots = slots.long()
        slots = slots.contiguous()
        if num_accepted_tokens is not None:
            if num_accepted_tokens.shape != (N,):
                raise ValueError(f'num_accepted_tokens must have shape ({N},), got {tuple(num_accepted_tokens.shape)}')
            accepted = num_accepted_tokens.to(device=dev, dtype=slots.dtype).contiguous()
        if not inplace_final_state:
            # read-only pool; the kernel finds the first slot the same way and returns a state per token
            per_token_out = True
            flags |= _lib.FLAG_STATE_PER_TOKEN
            if ssm_state_indices.ndim == 2:
                # (the start slot is picked on the host side of the kernel argument list: a gather of N indices)
                first = (accepted - 1) if accepted is not None else torch.zeros(N, dtype=slots.dtype, device=dev)
                slots = slots.gather(1, first.long()[:, None])[:, 0].to(slots.dtype).contiguous()
                accepted, slots_stride = None, 1
        state_shape = (h0.shape[0],) + state_shape[1:]            # the pool has its own number of slots
    if h0 is not None:
        if tuple(h0.shape) != state_shape:
            raise ValueError(f'initial_state must have shape {state_shape}, got {tuple(h0.shape)}')
        if inplace_final_state:
            if h0.dtype not in (torch.float32, torch.bfloat16) or h0.data_ptr() % 16 != 0:
                raise ValueError('inplace_final_state needs a contiguous, 16-byte aligned fp32 (or bf16) initial_state')
            if h0.dtype == torch.bfloat16:
                # states kept in bf16 between steps: half the traffic of a decode step; the step itself is fp32
                if ((K, V) != (128, 128) or state_v_first or gk is not None or gv is not None
                        or flags & (_lib.FLAG_BETA_VECTOR | _lib.FLAG_SLOT_PER_TOKEN)):
                    raise NotImplementedError('bf16 states need K = V = 128, the K-first layout, no gk / gv / beta per '
                                              'column and a state per sequence or per slot')
                flags |= _lib.FLAG_STATE_BF16
        else:
            h0 = aligned16(as_f32(h0))

    o = torch.empty_like(v)
    final_state = None
    if inplace_final_state:
        if initial_state is None:
            raise ValueError('inplace_final_state=True requires initial_state')
        final_state = h0
    elif per_token_out:
        final_state = torch.empty((B * T,) + state_shape[1:], dtype=torch.float32, device=dev)
    elif output_final_state:
        final_state = torch.empty(state_shape, dtype=torch.float32, device=dev)

    lib = _lib.load()
    if kda_gate_mode is not None:
        assert g is None and gv is None and gk is not None
        _lib.check(lib.gdn_fused_recurrent_kda_fwd(
            ptr(q), ptr(k), ptr(v), ptr(gk), ptr(beta), ptr(A_log), ptr(dt_bias), float(lower_bound), int(kda_gate_mode),
            ptr(h0), ptr(final_state), ptr(o), ptr(cu_seqlens), ptr(slots), ptr(accepted), slots_stride,
            B, T, H, HV, KP, VP, N, float(scale), dtype_code(q.dtype), gb_code, flags,
            current_stream_ptr(dev)))
    else:
        _lib.check(lib.gdn_fused_recurrent_fwd(
            ptr(q), ptr(k), ptr(v), ptr(g), ptr(beta), ptr(gk), ptr(gv), ptr(A_log), ptr(dt_bias),
            ptr(h0), ptr(final_state), ptr(o), ptr(cu_seqlens), ptr(slots), ptr(accepted), slots_stride,
            B, T, H, HV, KP, VP, N, float(scale), dtype_code(q.dtype), gb_code, flags,
            current_stream_ptr(dev)))
    if padded:
        o = o[..., :V].contiguous()
        if final_state is not None:
            final_state = (final_state[..., :V, :K] if state_v_first else final_state[..., :K, :V]).contiguous()
    return o, final_state


def fused_recurrent_gated_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor | None = None,
    gk: torch.Tensor | None = None,
    gv: torch.Tensor | None = None,
    beta: torch.Tensor | None = None,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    use_gate_in_kernel: bool = False,
    A_log: torch.Tensor | None = None,
    dt_bias: torch.Tensor | None = None,
    use_beta_sigmoid_in_kernel: bool = False,
    allow_neg_eigval: bool = False,
    state_v_first: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
    **kwargs,
) -> tuple[torch.Tensor, torch.Tensor]:
    r"""Token-by-token gated delta rule (decode / short prompts).

    Args:
        q, k: ``[B, T, H, K]``.  v: ``[B, T, HV, V]`` (``HV % H == 0``; each q/k head serves
            ``HV // H`` consecutive v heads).
        g: log-space decay ``[B, T, HV]``; raw pre-activation when ``use_gate_in_kernel``
            (then ``g = -exp(A_log) * softplus(g + dt_bias)`` is applied per step).
        gk / gv: optional per-key / per-value log decays ``[B, T, HV, K]`` / ``[B, T, HV, V]``.
        beta: ``[B, T, HV]`` (or ``[B, T, HV, V]``); ones when omitted; logits when
            ``use_beta_sigmoid_in_kernel`` (``allow_neg_eigval`` doubles the sigmoid).
        scale: defaults to ``K ** -0.5``.
        initial_state: ``[N, HV, K, V]`` (``[N, HV, V, K]`` when ``state_v_first``).
        output_final_state: also return the fp32 final state.
        cu_seqlens: ``[N + 1]`` int32/int64 boundaries of packed sequences (then ``B == 1``).
        inplace_final_state (keyword only, extension): write the final state over
            ``initial_state`` instead of allocating a new tensor.  A bf16 ``initial_state`` (K = V = 128, no
            ``gk`` / ``gv``) keeps the states in bf16 between calls: the step runs in fp32 and the state is rounded once,
            when it is written back, so a decode step moves half the bytes.
        ssm_state_indices (keyword only, extension; the sibling KDA operator's argument,
            fla/ops/kda/fused_recurrent.py:248-326): ``[N]`` int32/int64 slot of every sequence in the
            state pool ``initial_state [num_slots, HV, K, V]``; needs ``inplace_final_state=True``.
            Slots must be distinct; slots that are not named keep their contents.  ``[N, T]`` names a slot
            per token (speculative decoding, fla/ops/kda/fused_recurrent.py:131-145,203-219): the state after
            token t of sequence n goes to slot ``[n, t]``; without ``inplace_final_state`` the pool is only read
            and the states after every token are returned as ``[B * T, HV, K, V]``.
        num_accepted_tokens (keyword only, extension): ``[N]``; with ``ssm_state_indices [N, T]`` sequence n
            starts from slot ``[n, num_accepted_tokens[n] - 1]`` instead of ``[n, 0]``.

    Returns:
        ``(o [B, T, HV, V] in v's dtype, final_state or None)``.
    """
    if 'transpose_state_layout' in kwargs:
        if state_v_first:
            raise ValueError('Cannot pass both `state_v_first` and the deprecated `transpose_state_layout`.')
        warnings.warn('`transpose_state_layout` is deprecated and renamed to `state_v_first`.',
                      DeprecationWarning, stacklevel=2)
        state_v_first = kwargs.pop('transpose_state_layout')
    inplace_final_state = bool(kwargs.pop('inplace_final_state', False))
    ssm_state_indices = kwargs.pop('ssm_state_indices', None)
    num_accepted_tokens = kwargs.pop('num_accepted_tokens', None)

    if q.shape[2] != k.shape[2]:
        raise ValueError(f'q and k must have the same number of heads, got {q.shape[2]} and {k.shape[2]}')
    if v.shape[2] % q.shape[2] != 0:
        raise ValueError(f'num_v_heads (HV={v.shape[2]}) must be divisible by num_heads (H={q.shape[2]})')
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f'The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`.'
                f'Please flatten variable-length inputs before processing.')
        if initial_state is not None and ssm_state_indices is None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(
                f'The number of initial states is expected to be equal to the number of input sequences, '
                f'i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.')
    if scale is None:
        scale = k.shape[-1] ** -0.5
    if use_gate_in_kernel:
        if A_log is None:
            raise ValueError('`A_log` must be provided when `use_gate_in_kernel=True`.')
        if g is None:
            raise ValueError('`g` (raw pre-activation) must be provided when `use_gate_in_kernel=True`.')
    else:
        A_log = None
        dt_bias = None
    if allow_neg_eigval and not use_beta_sigmoid_in_kernel:
        raise ValueError('`allow_neg_eigval=True` requires `use_beta_sigmoid_in_kernel=True`.')
    if inplace_final_state and (initial_state is None or not initial_state.is_contiguous()
                                or initial_state.dtype not in (torch.float32, torch.bfloat16)):
        raise ValueError('`inplace_final_state=True` requires a contiguous fp32 (or bf16) `initial_state`.')

    return fused_recurrent_gated_delta_rule_fwd(
        q, k, v, g, gk, gv, beta, A_log, dt_bias, scale, initial_state, output_final_state,
        use_qk_l2norm_in_kernel, use_beta_sigmoid_in_kernel, allow_neg_eigval, state_v_first, cu_seqlens,
        inplace_final_state, ssm_state_indices, num_accepted_tokens)


fused_recurrent_gdn = fused_recurrent_gated_delta_rule
