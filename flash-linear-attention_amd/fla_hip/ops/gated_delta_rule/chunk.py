"""``chunk_gated_delta_rule``: same signature, defaults, validation and error types as
fla/ops/gated_delta_rule/chunk.py:397-593.  The reference's five Triton launches
(chunk.py:33-123) and its optional prologue launches (l2norm of q and k, gate activation,
beta sigmoid: chunk.py:278-288) are replaced by one call into libgdn_hip.so
(``gdn_chunk_fwd``), which runs a chunk-parallel HIP kernel (prologues, gate cumsum, gated
beta*K*K^T, 64x64 unit-lower solve, intra-chunk q k^T) and a sequential one (state
recurrence fused with the WY step and the output), so neither normalised copies of q and k
nor w, u or per-chunk states are ever written to memory."""
from __future__ import annotations

import os
import warnings

import torch

from fla_hip import _lib
from fla_hip.ops.backends import dispatch
from fla_hip.ops.gated_delta_rule._common import (
    check_operand_shapes,
    aligned16,
    as_f32,
    current_stream_ptr,
    dtype_code,
    ptr,
    require_gpu,
    unify_gate_beta,
)
from fla_hip.ops.utils.index import check_cu_seqlens, prepare_chunk_indices, prepare_scan_tables
from fla_hip.utils import input_guard

# The HIP kernels work on 64-token chunks.  The result of the operator does not depend on
# the chunk size (only rounding does), so chunk_size 16 and 32 are accepted and run with 64.
_KERNEL_CHUNK = 64
# FLA_HIP_SCAN_MODE forces one form of the sequential kernel (default: automatic): whole sequences
# ('wide') or time cut into segments, each with one run per workgroup ('-single') or two ('-pair')
_SCAN_MODE_FLAGS = {'wide': _lib.FLAG_SCAN_WIDE, 'segments': _lib.FLAG_SCAN_SEGMENTS,
                    'single': _lib.FLAG_SCAN_NO_PAIR, 'pair': _lib.FLAG_SCAN_PAIR,
                    'segments-exact': _lib.FLAG_SCAN_SEGMENTS | _lib.FLAG_SCAN_NO_WARM,
                    'record-p': _lib.FLAG_RECORD_P}       # (the prepare stage also writes P: for looking at its records)
for _form in ('wide', 'segments'):
    for _runs in ('single', 'pair'):
        _SCAN_MODE_FLAGS[f'{_form}-{_runs}'] = _SCAN_MODE_FLAGS[_form] | _SCAN_MODE_FLAGS[_runs]
        if _form == 'segments':
            _SCAN_MODE_FLAGS[f'segments-exact-{_runs}'] = _SCAN_MODE_FLAGS['segments-exact'] | _SCAN_MODE_FLAGS[_runs]
_KERNEL_DIMS = (128,)           # head dim the MFMA kernels are instantiated for (smaller dims are zero-padded)


def _pad_last(x: torch.Tensor, size: int) -> torch.Tensor:
    if x.shape[-1] == size:
        return x
    return torch.nn.functional.pad(x, (0, size - x.shape[-1]))


class ChunkLaunch:
    """Everything one forward call hands to the C ABI: normalised inputs, freshly allocated
    outputs and workspace, and the argument tuple of ``gdn_chunk_fwd``.  ``run()`` launches the
    whole operator; ``run('prepare')`` / ``run('scan')`` launch its two stages separately (same
    arguments), which is how the benchmark attributes time to each kernel."""

    _ENTRY = {None: 'gdn_chunk_fwd', 'prepare': 'gdn_chunk_fwd_prepare', 'scan': 'gdn_chunk_fwd_scan'}

    def __init__(self, q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first=False,
                 cu_seqlens=None, cu_seqlens_cpu=None, chunk_indices=None, chunk_size=64,
                 A_log=None, dt_bias=None, qk_l2norm=False, beta_sigmoid=False, neg_eigval=False):
        dev = require_gpu(q, k, v, beta) if g is None else require_gpu(q, k, v, g, beta)
        check_operand_shapes(q, k, v, g=g, beta=beta)
        B, T, H, K = k.shape
        HV, V = v.shape[2], v.shape[3]
        N = B if cu_seqlens is None else len(cu_seqlens) - 1
        self.out_dtype = q.dtype
        self.dims = (B, T, H, HV, K, V, N)
        self.state_v_first = state_v_first

        # the MFMA kernels take bf16 or fp16 operands; fp32 inputs are rounded to bf16 first
        work_dtype = q.dtype if q.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
        q, k, v = q.to(work_dtype), k.to(work_dtype), v.to(work_dtype)
        # The kernels take head dims that are multiples of 8 as they are.  Others are zero-padded
        # to the next one here: zero key features and zero value columns change neither the
        # other columns of the output nor the state entries that are kept.
        KP, VP = (K + 7) // 8 * 8, (V + 7) // 8 * 8
        self.padded = (KP, VP)
        q, k, v = _pad_last(q, KP), _pad_last(k, KP), _pad_last(v, VP)
        g, beta, gb_code = unify_gate_beta(g, beta)

        flags = _lib.FLAG_STATE_V_FIRST if state_v_first else 0
        # prologues the kernels apply themselves
        if qk_l2norm:
            flags |= _lib.FLAG_QK_L2NORM
        if beta_sigmoid:
            flags |= _lib.FLAG_BETA_SIGMOID | (_lib.FLAG_NEG_EIGVAL if neg_eigval else 0)
        if A_log is not None:
            A_log = A_log.detach().to(device=dev, dtype=torch.float32).contiguous()
            if A_log.numel() != HV:
                raise ValueError(f'A_log must have {HV} entries, got {A_log.numel()}')
        if dt_bias is not None:
            dt_bias = dt_bias.detach().to(device=dev, dtype=torch.float32).contiguous()
            if dt_bias.numel() != HV:
                raise ValueError(f'dt_bias must have {HV} entries, got {dt_bias.numel()}')
        flags |= _SCAN_MODE_FLAGS.get(os.environ.get('FLA_HIP_SCAN_MODE', 'auto'), 0)
        if cu_seqlens is not None:
            if cu_seqlens.dtype not in (torch.int32, torch.int64):
                cu_seqlens = cu_seqlens.long()
            if cu_seqlens.device != dev:
                cu_seqlens = cu_seqlens.to(dev)
            if cu_seqlens.dtype == torch.int32:
                flags |= _lib.FLAG_CU_INT32
            check_cu_seqlens(cu_seqlens, T, cu_seqlens_cpu)
            # (a caller's chunk_indices are not taken over: the kernels index with them, so they are derived here from the
            # boundaries just checked - memoised per cu_seqlens tensor, as the reference's are)
            chunk_indices = prepare_chunk_indices(cu_seqlens, _KERNEL_CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)
            chunk_indices = chunk_indices.to(device=dev, dtype=cu_seqlens.dtype).contiguous()
            # chunk offsets per sequence, followed by the longest-first order of the sequences
            chunk_offsets = prepare_scan_tables(cu_seqlens, _KERNEL_CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)
            flags |= _lib.FLAG_SEQ_ORDER
            num_chunks = chunk_indices.shape[0]
        else:
            chunk_indices = chunk_offsets = None
            num_chunks = B * ((T + _KERNEL_CHUNK - 1) // _KERNEL_CHUNK)

        state_shape = (N, HV, V, K) if state_v_first else (N, HV, K, V)
        h0 = initial_state
        if h0 is not None:
            if tuple(h0.shape) != state_shape:
                raise ValueError(f'initial_state must have shape {state_shape}, got {tuple(h0.shape)}')
            h0 = as_f32(h0)
            if (KP, VP) != (K, V):
                h0 = torch.nn.functional.pad(h0, (0, (KP if state_v_first else VP) - h0.shape[-1],
                                                  0, (VP if state_v_first else KP) - h0.shape[-2]))
            h0 = aligned16(h0.contiguous())

        self.o = torch.empty(B, T, HV, VP, dtype=work_dtype, device=dev)
        self.ht = None
        if output_final_state:
            self.ht = torch.empty((N, HV, VP, KP) if state_v_first else (N, HV, KP, VP), dtype=torch.float32, device=dev)
        self.h0 = h0

        self.lib = _lib.load()
        ws_bytes = self.lib.gdn_chunk_workspace_bytes(N, T, num_chunks, H, HV, KP, VP, int(cu_seqlens is not None), flags)
        if ws_bytes == 0 and num_chunks > 0:
            raise NotImplementedError(f'HIP chunk kernels do not cover K={KP}, V={VP}')
        self.workspace = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
        self.keep = (q, k, v, g, beta, A_log, dt_bias, cu_seqlens, chunk_indices, chunk_offsets)     # keep the buffers alive
        self.device = dev
        self.args = (
            ptr(q), ptr(k), ptr(v), ptr(g), ptr(beta), ptr(A_log), ptr(dt_bias), ptr(h0), ptr(self.ht), ptr(self.o),
            ptr(cu_seqlens), ptr(chunk_indices), ptr(chunk_offsets),
            ptr(self.workspace), ws_bytes,
            B, T, H, HV, KP, VP, N, num_chunks,
            float(scale), dtype_code(work_dtype), gb_code, flags)

    def run(self, stage: str | None = None) -> None:
        fn = getattr(self.lib, self._ENTRY[stage])          # (without tokens the library copies h0 into ht)
        _lib.check(fn(*self.args, current_stream_ptr(self.device)))

    def results(self) -> tuple[torch.Tensor, torch.Tensor | None]:
        B, T, H, HV, K, V, N = self.dims
        KP, VP = self.padded
        o, ht = self.o, self.ht
        if VP != V:
            o = o[..., :V]
        if ht is not None and (KP, VP) != (K, V):
            ht = (ht[..., :V, :K] if self.state_v_first else ht[..., :K, :V]).contiguous()
        return o.to(self.out_dtype), ht


@input_guard
def chunk_gated_delta_rule_fwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    scale: float,
    initial_state: torch.Tensor | None,
    output_final_state: bool,
    state_v_first: bool = False,
    cu_seqlens: torch.Tensor | None = None,
    cu_seqlens_cpu: torch.Tensor | None = None,
    chunk_indices: torch.Tensor | None = None,
    chunk_size: int = 64,
    A_log: torch.Tensor | None = None,
    dt_bias: torch.Tensor | None = None,
    use_qk_l2norm_in_kernel: bool = False,
    use_beta_sigmoid_in_kernel: bool = False,
    allow_neg_eigval: bool = False,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Forward of the chunked operator.  ``g`` is the log-space decay (raw gate inputs when
    ``A_log`` is given), ``beta`` the write strength (logits with ``use_beta_sigmoid_in_kernel``).
    Returns ``(o in q's dtype, final_state fp32 or None)``."""
    K, V = k.shape[-1], v.shape[-1]
    assert K <= 256, 'current kernel does not support head dimension larger than 256.'     # (chunk_delta_h.py:712)
    # Wide keys (128 < K <= 256) have a scan kernel of their own that takes any number of value columns, 64 per workgroup.
    nb = (V + _KERNEL_DIMS[-1] - 1) // _KERNEL_DIMS[-1] if K <= _KERNEL_DIMS[-1] else 1
    if nb > 1:
        # The value columns of the recurrence are independent: a head with V > 128 is nb heads of 128
        # columns that share the head's k, q, gate and beta (grouped value heads do exactly that).
        D = _KERNEL_DIMS[-1]
        B, T, HV = v.shape[:3]
        N = B if cu_seqlens is None else len(cu_seqlens) - 1
        v2 = _pad_last(v, nb * D).reshape(B, T, HV * nb, D)
        g2, beta2 = None if g is None else g.repeat_interleave(nb, dim=2), beta.repeat_interleave(nb, dim=2)
        A2 = None if A_log is None else A_log.reshape(-1).repeat_interleave(nb)
        dt2 = None if dt_bias is None else dt_bias.reshape(-1).repeat_interleave(nb)
        h2 = None
        if initial_state is not None:
            if state_v_first:       # [N, HV, V, K] -> [N, HV*nb, D, K]
                h2 = torch.nn.functional.pad(initial_state, (0, 0, 0, nb * D - V)).reshape(N, HV * nb, D, K)
            else:                   # [N, HV, K, V] -> [N, HV*nb, K, D]
                h2 = _pad_last(initial_state, nb * D).reshape(N, HV, K, nb, D).permute(0, 1, 3, 2, 4).reshape(N, HV * nb, K, D)
        o2, ht2 = chunk_gated_delta_rule_fwd(
            q, k, v2, g2, beta2, scale, h2, output_final_state, state_v_first, cu_seqlens, cu_seqlens_cpu,
            chunk_indices, chunk_size, A2, dt2, use_qk_l2norm_in_kernel, use_beta_sigmoid_in_kernel, allow_neg_eigval)
        o = o2.reshape(B, T, HV, nb * D)[..., :V]
        ht = None
        if ht2 is not None:
            if state_v_first:
                ht = ht2.reshape(N, HV, nb * D, K)[:, :, :V]
            else:
                ht = ht2.reshape(N, HV, nb, K, D).permute(0, 1, 3, 2, 4).reshape(N, HV, K, nb * D)[..., :V]
            ht = ht.contiguous()
        return o.contiguous() if nb * D != V else o, ht
    call = ChunkLaunch(q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first,
                       cu_seqlens, cu_seqlens_cpu, chunk_indices, chunk_size,
                       A_log, dt_bias, use_qk_l2norm_in_kernel, use_beta_sigmoid_in_kernel, allow_neg_eigval)
    call.run()
    return call.results()


@dispatch('gated_delta_rule')
@torch.compiler.disable
def chunk_gated_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    scale: float | None = None,
    initial_state: torch.Tensor | None = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    use_beta_sigmoid_in_kernel: bool = False,
    allow_neg_eigval: bool = False,
    state_v_first: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
    cu_seqlens_cpu: torch.LongTensor | None = None,
    chunk_indices: torch.LongTensor | None = None,
    cp_context=None,
    **kwargs,
):
    r"""Chunked gated delta rule (prefill; differentiable: inputs that require a gradient get one).

    Args:
        q, k: ``[B, T, H, K]``.  v: ``[B, T, HV, V]`` with ``HV % H == 0`` (grouped value heads).
        g: log-space decay ``[B, T, HV]`` (raw pre-activation with ``use_gate_in_kernel=True``,
            ``A_log`` and optional ``dt_bias`` passed as keywords).
        beta: ``[B, T, HV]`` (logits with ``use_beta_sigmoid_in_kernel=True``;
            ``allow_neg_eigval`` doubles the sigmoid).
        scale: defaults to ``K ** -0.5``.
        initial_state: ``[N, HV, K, V]`` (``[N, HV, V, K]`` with ``state_v_first``), any float dtype.
        output_final_state: also return the fp32 final state.
        use_qk_l2norm_in_kernel: L2-normalise q and k per head first.
        cu_seqlens: ``[N + 1]`` int32/int64 boundaries of packed sequences (then ``B == 1``);
            ``cu_seqlens_cpu`` is an optional host copy that avoids a device sync;
            ``chunk_indices`` optional precomputed chunk table for ``chunk_size``.
        cp_context: context parallelism is not part of this single-GPU build.

    Returns:
        ``(o [B, T, HV, V] in q's dtype, final_state or None)``.
    """
    if 'transpose_state_layout' in kwargs:
        if state_v_first:
            raise ValueError('Cannot pass both `state_v_first` and the deprecated `transpose_state_layout`.')
        warnings.warn('`transpose_state_layout` is deprecated and renamed to `state_v_first`.',
                      DeprecationWarning, stacklevel=2)
        state_v_first = kwargs.pop('transpose_state_layout')

    if q.shape[2] != k.shape[2]:
        raise ValueError(
            f'q and k must have the same number of heads, '
            f'but got q.shape[2]={q.shape[2]} and k.shape[2]={k.shape[2]}')
    H, HV = q.shape[2], v.shape[2]
    if HV % H != 0:
        raise ValueError(
            f'For GVA, num_v_heads (HV={HV}) must be evenly divisible by '
            f'num_heads (H={H}), but got HV % H = {HV % H}')
    if 'head_first' in kwargs:
        raise DeprecationWarning('head_first has been removed. Inputs must be in `[B, T, H, ...]` format.')
    chunk_size = kwargs.pop('chunk_size', 64)
    if chunk_size not in (16, 32, 64):
        raise ValueError(f'`chunk_size` must be 16, 32, or 64 for Gated Delta Rule, got {chunk_size}.')
    if cp_context is not None:
        raise NotImplementedError('context parallelism (cp_context) is outside this single-GPU build')
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f'The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`.'
                f'Please flatten variable-length inputs before processing.')
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(
                f'The number of initial states is expected to be equal to the number of input sequences, '
                f'i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.')
    use_gate_in_kernel = kwargs.get('use_gate_in_kernel', False)
    A_log = kwargs.get('A_log')
    dt_bias = kwargs.get('dt_bias')
    if use_gate_in_kernel:
        assert A_log is not None, 'A_log must be provided when use_gate_in_kernel=True.'
    if allow_neg_eigval and not use_beta_sigmoid_in_kernel:
        raise ValueError('`allow_neg_eigval=True` requires `use_beta_sigmoid_in_kernel=True`.')
    if scale is None:
        scale = k.shape[-1] ** -0.5

    if torch.is_grad_enabled() and any(
            x is not None and x.requires_grad for x in (q, k, v, g, beta, initial_state, A_log, dt_bias)):
        # training: the same forward kernels inside an autograd function (chunk.py:260-395)
        from fla_hip.ops.gated_delta_rule.chunk_bwd import ChunkGatedDeltaRuleFunction
        return ChunkGatedDeltaRuleFunction.apply(
            q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first, cu_seqlens, cu_seqlens_cpu,
            chunk_indices, use_qk_l2norm_in_kernel, use_gate_in_kernel, A_log, dt_bias,
            use_beta_sigmoid_in_kernel, allow_neg_eigval, chunk_size)
    # the prologues the reference runs as separate launches before its chunk pipeline
    # (chunk.py:278-288, gate.py:63-106) happen inside the first kernel
    return chunk_gated_delta_rule_fwd(
        q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first,
        cu_seqlens, cu_seqlens_cpu, chunk_indices, chunk_size,
        A_log if use_gate_in_kernel else None, dt_bias if use_gate_in_kernel else None,
        use_qk_l2norm_in_kernel, use_beta_sigmoid_in_kernel, allow_neg_eigval)


chunk_gdn = chunk_gated_delta_rule
