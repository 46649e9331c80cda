"""``chunk_comba``: chunked prefill of the comba operator (the gated delta rule whose prediction uses a second key ``p`` and
the state before the token's decay), with the signature and validation of fla/ops/comba/chunk.py:292-406.
The reference's forward launches (``chunk_comba_cumsum_scalar_fwd``, ``chunk_scaled_dot_comba_pkt_fwd``, the triangular
solve, ``recompute_w_u_fwd``, ``chunk_gated_delta_rule_fwd_h``, ``chunk_fwd_o``; fla/ops/comba/chunk.py:22-90) are one call
into libgdn_hip.so (``gdn_chunk_comba_fwd``): a chunk-parallel kernel and the sequential kernel of the chunked KDA forward.
Its backward (``chunk_comba_bwd``, chunk.py:92-178, inside ``ChunkCombaFunction``, :181-289) is one call as well
(``gdn_chunk_comba_bwd``): the kernels of the gated delta rule's backward, two of them in their comba form; nothing is
kept from the forward call but its inputs."""
from __future__ import annotations

import torch
import torch.nn.functional as F

from fla_hip import _lib
from fla_hip.ops.gated_delta_rule._common import (
    pad_last_two,
    aligned16,
    check_operand_shapes,
    as_f32,
    current_stream_ptr,
    dtype_code,
    ptr,
    require_gpu,
)
from fla_hip.ops.gated_delta_rule.chunk_bwd import _finish, l2norm_fwd
from fla_hip.ops.utils.index import check_cu_seqlens, cu_bounds, prepare_chunk_indices, prepare_scan_tables

_CHUNK = 64
_DIM = 128          # head dims of the kernels; smaller ones are zero-padded


def _pad_last(x: torch.Tensor, size: int) -> torch.Tensor:
    return x if x.shape[-1] == size else F.pad(x, (0, size - x.shape[-1]))


def chunk_comba_fwd(q, k, v, p, g, beta, scale, initial_state, output_final_state, use_qk_l2norm_in_kernel=False,
                    cu_seqlens=None, cu_seqlens_cpu=None, fp32_as=torch.bfloat16):
    """Returns ``(o [B,T,HV,V] in q's dtype, final_state [N,HV,K,V] fp32 or None)``.  The kernels take 16-bit operands
    (the state and all sums are fp32); inputs of another dtype are converted to ``fp32_as`` first."""
    dev = require_gpu(q, k, v, p, g, beta)
    check_operand_shapes(q, k, v, g=g, beta=beta)
    if p.shape != q.shape:
        raise ValueError(f'q, k and p must share one shape, got {tuple(q.shape)}, {tuple(k.shape)}, {tuple(p.shape)}')
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if K > _DIM:
        # Wide keys: the chunked kernels hold one block of 128 key features, so the forward goes token by token on the
        # recurrence kernel, which holds two (the same mathematics, far slower on long prompts); no backward at this width.
        if K > 2 * _DIM:
            raise NotImplementedError(f'chunk_comba covers key head dims up to {2 * _DIM} (got K={K})')
        from fla_hip.ops.comba.fused_recurrent import fused_recurrent_comba_fwd
        o, ht = fused_recurrent_comba_fwd(q, k, p, v, g, beta, scale, initial_state, output_final_state, use_qk_l2norm_in_kernel,
                                          cu_seqlens)
        return o.to(q.dtype), ht
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    nb = (V + _DIM - 1) // _DIM
    if nb > 1:
        # value columns are independent: a head with V > 128 is nb heads of 128 columns that share q, k, p, g, beta
        v2 = _pad_last(v, nb * _DIM).reshape(B, T, HV * nb, _DIM)
        h2 = None
        if initial_state is not None:
            h2 = _pad_last(initial_state, nb * _DIM).reshape(N, HV, K, nb, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV * nb, K, _DIM)
        o2, ht2 = chunk_comba_fwd(q, k, v2, p, g.repeat_interleave(nb, dim=2), beta.repeat_interleave(nb, dim=2), scale, h2,
                                  output_final_state, use_qk_l2norm_in_kernel, cu_seqlens, cu_seqlens_cpu, fp32_as)
        o = o2.reshape(B, T, HV, nb * _DIM)[..., :V].contiguous()
        ht = None
        if ht2 is not None:
            ht = ht2.reshape(N, HV, nb, K, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV, K, nb * _DIM)[..., :V].contiguous()
        return o, ht

    out_dtype = q.dtype
    work = q.dtype if q.dtype in (torch.bfloat16, torch.float16) else fp32_as
    qw, kw, vw, pw = (aligned16(_pad_last(x.to(work), _DIM).contiguous()) for x in (q, k, v, p))
    gw, bw = as_f32(g).contiguous(), as_f32(beta).contiguous()
    h0 = None
    if initial_state is not None:
        if tuple(initial_state.shape) != (N, HV, K, V):
            raise ValueError(f'initial_state must have shape {(N, HV, K, V)}, got {tuple(initial_state.shape)}')
        h0 = aligned16(pad_last_two(as_f32(initial_state), _DIM, _DIM).contiguous())

    flags = _lib.FLAG_QK_L2NORM if use_qk_l2norm_in_kernel else 0
    chunk_table = chunk_offsets = None
    if cu_seqlens is not None:
        if cu_seqlens.dtype not in (torch.int32, torch.int64):
            cu_seqlens = cu_seqlens.long()
        cu_seqlens = cu_seqlens.to(dev)
        if cu_seqlens.dtype == torch.int32:
            flags |= _lib.FLAG_CU_INT32
        check_cu_seqlens(cu_seqlens, T, cu_seqlens_cpu)
        chunk_table = prepare_chunk_indices(cu_seqlens, _CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)
        chunk_table = chunk_table.to(device=dev, dtype=cu_seqlens.dtype).contiguous()
        chunk_offsets = prepare_scan_tables(cu_seqlens, _CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)
        num_chunks = chunk_table.shape[0]
    else:
        num_chunks = B * ((T + _CHUNK - 1) // _CHUNK)

    o = torch.empty(B, T, HV, _DIM, dtype=work, device=dev)
    ht = torch.empty(N, HV, _DIM, _DIM, dtype=torch.float32, device=dev) if output_final_state else None
    lib = _lib.load()
    ws_bytes = lib.gdn_chunk_kda_workspace_bytes(num_chunks, HV)
    workspace = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    _lib.check(lib.gdn_chunk_comba_fwd(
        ptr(qw), ptr(kw), ptr(vw), ptr(pw), ptr(gw), ptr(bw), ptr(h0), ptr(ht), ptr(o),
        ptr(cu_seqlens), ptr(chunk_table), ptr(chunk_offsets), ptr(workspace), ws_bytes,
        B, T, H, HV, _DIM, _DIM, N, num_chunks, float(scale), dtype_code(work), _lib.DTYPE_F32, flags,
        current_stream_ptr(dev)))
    o = o[..., :V].to(out_dtype)
    if ht is not None:
        ht = ht[..., :K, :V].contiguous()
    return o, ht


def chunk_comba_bwd(q, k, v, p, g, beta, scale, initial_state, do, dht, cu_seqlens=None, cu_seqlens_cpu=None,
                    q_rstd=None, k_rstd=None, p_rstd=None, qk_l2norm=False):
    """q, k, p ``[B,T,H,K]``, v, do ``[B,T,HV,V]``, g (log decay), beta ``[B,T,HV]`` as the recurrence uses them.
    Returns ``(dq, dk, dv, dp, dbeta, dg, dh0)``: dq, dk, dv, dp in q's dtype, dbeta, dg fp32, dh0 fp32 (None without
    ``initial_state``).  With the ``*_rstd`` factors (what ``l2norm_fwd`` returns next to the normalised rows passed as
    q, k, p) dq, dk, dp are the gradients of the rows before normalisation (fla/ops/comba/chunk.py:277-280).  With
    ``qk_l2norm`` q, k, p are the rows BEFORE their l2 normalisation and dq, dk, dp the gradients of those: one C call
    (``gdn_chunk_comba_bwd_qk_l2norm``) where every value head has a q/k head of its own, ``l2norm_fwd`` and the route above
    otherwise."""
    dev = require_gpu(q, k, v, p, g, beta, do)
    check_operand_shapes(q, k, v, g=g, beta=beta)
    if do.shape != v.shape:
        raise ValueError(f'do must have the shape of v, got {tuple(do.shape)} and {tuple(v.shape)}')
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if K > _DIM:
        raise NotImplementedError(f'the chunked comba kernels cover key head dims up to {_DIM} (got K={K})')
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    nb = (V + _DIM - 1) // _DIM
    inside = qk_l2norm and H == HV and nb == 1
    if qk_l2norm and not inside:
        (q, q_rstd), (k, k_rstd), (p, p_rstd) = l2norm_fwd(q), l2norm_fwd(k), l2norm_fwd(p)
        q, k, p = (x[..., :K] for x in (q, k, p))          # (l2norm_fwd pads rows to a multiple of 8)
    if nb > 1:
        # value columns are independent: a head with V > 128 is nb heads of 128 columns that share q, k, p, g, beta
        def split(s):       # [N, HV, K, V] -> [N, HV*nb, K, 128]
            if s is None:
                return None
            return _pad_last(s, nb * _DIM).reshape(N, HV, K, nb, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV * nb, K, _DIM)
        v2 = _pad_last(v, nb * _DIM).reshape(B, T, HV * nb, _DIM)
        do2 = _pad_last(do, nb * _DIM).reshape(B, T, HV * nb, _DIM)
        dq, dk, dv2, dp, db2, dg2, dh2 = chunk_comba_bwd(
            q, k, v2, p, g.repeat_interleave(nb, dim=2), beta.repeat_interleave(nb, dim=2), scale, split(initial_state), do2,
            split(dht), cu_seqlens, cu_seqlens_cpu, q_rstd, k_rstd, p_rstd)
        dv = dv2.reshape(B, T, HV, nb * _DIM)[..., :V].contiguous()
        db, dg = db2.reshape(B, T, HV, nb).sum(-1), dg2.reshape(B, T, HV, nb).sum(-1)
        dh0 = None
        if dh2 is not None:
            dh0 = dh2.reshape(N, HV, nb, K, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV, K, nb * _DIM)[..., :V].contiguous()
        return dq, dk, dv, dp, db, dg, dh0

    out_dtype = q.dtype
    work = q.dtype if q.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    qw, kw, pw, vw, dow = (aligned16(_pad_last(x.to(work), _DIM).contiguous()) for x in (q, k, p, v, do))
    gw, bw = as_f32(g).contiguous(), as_f32(beta).contiguous()

    def state_in(s):
        if s is None:
            return None
        if tuple(s.shape) != (N, HV, K, V):
            raise ValueError(f'initial_state and dht must have shape {(N, HV, K, V)}, got {tuple(s.shape)}')
        return aligned16(pad_last_two(as_f32(s), _DIM, _DIM).contiguous())
    h0, dhtw = state_in(initial_state), state_in(dht)

    flags = 0
    chunk_table = chunk_offsets = None
    alloc = torch.empty
    if cu_seqlens is not None:
        if cu_seqlens.dtype not in (torch.int32, torch.int64):
            cu_seqlens = cu_seqlens.long()
        cu_seqlens = cu_seqlens.to(dev)
        if cu_seqlens.dtype == torch.int32:
            flags |= _lib.FLAG_CU_INT32
        check_cu_seqlens(cu_seqlens, T, cu_seqlens_cpu)
        chunk_table = prepare_chunk_indices(cu_seqlens, _CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)
        chunk_table = chunk_table.to(device=dev, dtype=cu_seqlens.dtype).contiguous()
        chunk_offsets = prepare_scan_tables(cu_seqlens, _CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)
        num_chunks = chunk_table.shape[0]
        # tokens of a packed tensor outside every sequence are never written: they get zero gradients
        first, last = cu_bounds(cu_seqlens, cu_seqlens_cpu)
        if first != 0 or last != T:
            alloc = torch.zeros
    else:
        num_chunks = B * ((T + _CHUNK - 1) // _CHUNK)

    dq, dk, dp = (alloc(B, T, HV, _DIM, dtype=work, device=dev) for _ in range(3))
    dv = alloc(B, T, HV, _DIM, dtype=work, device=dev)
    dg = alloc(B, T, HV, dtype=torch.float32, device=dev)
    db = alloc(B, T, HV, dtype=torch.float32, device=dev)
    dh0 = torch.empty(N, HV, _DIM, _DIM, dtype=torch.float32, device=dev) if initial_state is not None else None
    lib = _lib.load()
    ws_bytes = lib.gdn_chunk_comba_bwd_qk_l2norm_workspace_bytes(num_chunks, HV, B * T) if inside else lib.gdn_chunk_bwd_workspace_bytes(num_chunks, HV, _DIM)
    workspace = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    _lib.check((lib.gdn_chunk_comba_bwd_qk_l2norm if inside else lib.gdn_chunk_comba_bwd)(
        ptr(qw), ptr(kw), ptr(pw), ptr(vw), ptr(gw), ptr(bw), ptr(h0), ptr(dow), ptr(dhtw),
        ptr(dq), ptr(dk), ptr(dp), ptr(dv), ptr(dg), ptr(db), ptr(dh0),
        ptr(cu_seqlens), ptr(chunk_table), ptr(chunk_offsets), ptr(workspace), ws_bytes,
        B, T, H, HV, _DIM, _DIM, N, num_chunks, float(scale), dtype_code(work), _lib.DTYPE_F32, flags,
        current_stream_ptr(dev)))
    dq = _finish(lib, dq, qw, q_rstd, H, K, out_dtype)
    dk = _finish(lib, dk, kw, k_rstd, H, K, out_dtype)
    dp = _finish(lib, dp, pw, p_rstd, H, K, out_dtype)
    dv = dv[..., :V].to(out_dtype)
    if dh0 is not None:
        dh0 = dh0[..., :K, :V].contiguous()
    return dq, dk, dv, dp, db, dg, dh0


class ChunkCombaFunction(torch.autograd.Function):
    """Forward through ``gdn_chunk_comba_fwd``, backward through ``gdn_chunk_comba_bwd`` (fla/ops/comba/chunk.py:181-289)."""

    @staticmethod
    def forward(ctx, q, k, v, p, g, beta, scale, initial_state, output_final_state, use_qk_l2norm_in_kernel, cu_seqlens,
                cu_seqlens_cpu):
        o, ht = chunk_comba_fwd(q, k, v, p, g, beta, scale, initial_state, output_final_state, use_qk_l2norm_in_kernel,
                                cu_seqlens, cu_seqlens_cpu)
        ctx.save_for_backward(q, k, v, p, g, beta, initial_state, cu_seqlens, cu_seqlens_cpu)
        ctx.opts = (scale, use_qk_l2norm_in_kernel)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        q, k, v, p, g, beta, h0, cu_seqlens, cu_seqlens_cpu = ctx.saved_tensors
        scale, l2 = ctx.opts
        dq, dk, dv, dp, db, dg, dh0 = chunk_comba_bwd(q, k, v, p, g, beta, scale, h0, do.contiguous(), dht, cu_seqlens,
                                                      cu_seqlens_cpu, qk_l2norm=l2)
        K = q.shape[-1]
        return (dq[..., :K].to(q.dtype), dk[..., :K].to(k.dtype), dv.to(v.dtype), dp[..., :K].to(p.dtype), dg.to(g.dtype),
                db.to(beta.dtype), None, dh0, None, None, None, None)


def check_comba_args(q, k, v, p, g, beta, initial_state, cu_seqlens):
    """The reference's checks (fla/ops/comba/chunk.py:376-388) and the shapes the kernels rely on."""
    if cu_seqlens is not None:
        if q.shape[0] != 1:
            raise ValueError(
                f'The batch size is expected to be 1 rather than {q.shape[0]} when using `cu_seqlens`.'
                f'Please flatten variable-length inputs before processing.')
        if initial_state is not None and initial_state.shape[0] != len(cu_seqlens) - 1:
            raise ValueError(
                f'The number of initial states is expected to be equal to the number of input sequences, '
                f'i.e., {len(cu_seqlens) - 1} rather than {initial_state.shape[0]}.')
    H, HV = q.shape[2], v.shape[2]
    if k.shape != q.shape or p.shape != q.shape:
        raise ValueError(f'q, k and p must share one shape, got {tuple(q.shape)}, {tuple(k.shape)}, {tuple(p.shape)}')
    if HV % H != 0:
        raise ValueError(f'HV={HV} must be a multiple of H={H}')
    if g.shape != v.shape[:3] or beta.shape != v.shape[:3]:
        raise ValueError(f'g and beta must have shape {tuple(v.shape[:3])}, got {tuple(g.shape)} and {tuple(beta.shape)}')


@torch.compiler.disable
def chunk_comba(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    p: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor = None,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
    cu_seqlens_cpu: torch.LongTensor | None = None,
):
    r"""Chunked comba (prefill); differentiable in q, k, v, p, g, beta and ``initial_state``.

    Args:
        q, k, p: ``[B, T, H, K]``; ``p`` (the key the prediction is made with) defaults to ``k``.
        v: ``[B, T, HV, V]`` with ``HV % H == 0``.
        g: ``[B, T, HV]`` decays in log space; beta: ``[B, T, HV]`` (ones when ``None``).
        scale: defaults to ``K ** -0.5``.  initial_state: ``[N, HV, K, V]``.
        use_qk_l2norm_in_kernel: normalise q, k and p inside the kernel.
        cu_seqlens: ``[N + 1]`` boundaries of packed sequences (then ``B == 1``).

    Returns:
        ``(o [B, T, HV, V] in q's dtype, final_state [N, HV, K, V] fp32 or None)``.
    """
    if p is None:
        p = k
    if beta is None:
        beta = torch.ones_like(g)
    check_comba_args(q, k, v, p, g, beta, initial_state, cu_seqlens)
    if scale is None:
        scale = k.shape[-1] ** -0.5
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in (q, k, v, p, g, beta, initial_state)):
        if k.shape[-1] > _DIM:
            raise NotImplementedError(f'chunk_comba with key head dims above {_DIM} is forward only (got K={k.shape[-1]})')
        return ChunkCombaFunction.apply(q, k, v, p, g, beta, scale, initial_state, output_final_state,
                                        use_qk_l2norm_in_kernel, cu_seqlens, cu_seqlens_cpu)
    return chunk_comba_fwd(q, k, v, p, g, beta, scale, initial_state, output_final_state, use_qk_l2norm_in_kernel,
                           cu_seqlens, cu_seqlens_cpu)
