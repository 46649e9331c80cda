"""Backward of ``chunk_gated_delta_rule``: ``chunk_gated_delta_rule_bwd`` with the argument meaning of
fla/ops/gated_delta_rule/chunk.py:125-257 and the autograd function around forward and backward
(chunk.py:260-395).  One call into libgdn_hip.so (``gdn_chunk_bwd``) replaces the reference's seven launches;
nothing is kept from the forward call but its inputs (A, w, u, the per-chunk states and v_new are computed
again).  The activations the forward kernels apply themselves (l2 norm of q and k, gate, beta sigmoid) and
their derivatives are elementwise work around that call, as in the reference (chunk.py:278-288, 385-393)."""
from __future__ import annotations

import os

import torch
import torch.nn.functional as F

from fla_hip import _lib
from fla_hip.ops.gated_delta_rule._common import aligned16, as_f32, check_operand_shapes, current_stream_ptr, dtype_code, pad_last_two, ptr, require_gpu
from fla_hip.ops.utils.index import check_cu_seqlens, cu_bounds, prepare_chunk_indices, prepare_scan_tables

_CHUNK = 64
_DIM = 128          # value columns of the backward kernels; key features: 128 or 256 (other head dims are zero-padded)


def _pad_last(x: torch.Tensor, size: int) -> torch.Tensor:
    return x if x.shape[-1] == size else F.pad(x, (0, size - x.shape[-1]))


def chunk_gated_delta_rule_bwd(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor | None,
    beta: torch.Tensor,
    scale: float,
    initial_state: torch.Tensor | None,
    do: torch.Tensor,
    dht: torch.Tensor | None,
    state_v_first: bool = False,
    cu_seqlens: torch.Tensor | None = None,
    cu_seqlens_cpu: torch.Tensor | None = None,
    chunk_indices: torch.Tensor | None = None,
    chunk_size: int = 64,
    q_rstd: torch.Tensor | None = None,
    k_rstd: torch.Tensor | None = None,
    qk_l2norm: bool = False,
):
    """q, k ``[B,T,H,K]``, v, do ``[B,T,HV,V]``, g (log decay), beta ``[B,T,HV]`` as the recurrence uses them.
    Returns ``(dq, dk, dv, dbeta, dg, dh0)``: dq, dk, dv in q's dtype, dbeta, dg fp32, dh0 fp32 (None without
    ``initial_state``).  With ``q_rstd``, ``k_rstd`` (the factors ``l2norm_fwd`` returns next to the normalised rows
    passed as q and k) dq and dk are the gradients of the rows before normalisation: the reference's ``l2norm_bwd``
    (chunk.py:385-387) happens in the kernel that also adds up the value heads of a q/k head.  With ``qk_l2norm`` q and k
    are the rows BEFORE their l2 normalisation and dq, dk the gradients of those: one C call (``gdn_chunk_bwd_qk_l2norm``)
    where every value head has a q/k head of its own and K <= 128, ``l2norm_fwd`` and the route above otherwise."""
    dev = require_gpu(q, k, v, beta, do)
    check_operand_shapes(q, k, v, g=g, beta=beta)
    if do.shape != v.shape:
        raise ValueError(f'do must have the shape of v, got {tuple(do.shape)} and {tuple(v.shape)}')
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if K > 2 * _DIM:
        raise NotImplementedError(f'the backward kernels cover key head dims up to {2 * _DIM} (got K={K})')
    KD = _DIM if K <= _DIM else 2 * _DIM
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    inside = qk_l2norm and H == HV and KD == _DIM and V <= _DIM
    if qk_l2norm and not inside:
        q, q_rstd = l2norm_fwd(q)
        k, k_rstd = l2norm_fwd(k)
        q, k = q[..., :K], k[..., :K]                  # (l2norm_fwd pads rows to a multiple of 8)
    nb = (V + _DIM - 1) // _DIM
    if nb > 1:
        # value columns are independent: a head with V > 128 is nb heads of 128 columns that share q, k, g, beta
        v2 = _pad_last(v, nb * _DIM).reshape(B, T, HV * nb, _DIM)
        do2 = _pad_last(do, nb * _DIM).reshape(B, T, HV * nb, _DIM)
        g2 = None if g is None else g.repeat_interleave(nb, dim=2)
        h2 = d2 = None

        def split(s):       # [N, HV, K, V] -> [N, HV*nb, K, 128]  (V-first: [N, HV, V, K] -> [N, HV*nb, 128, K])
            if s is None:
                return None
            if state_v_first:
                return F.pad(s, (0, 0, 0, nb * _DIM - V)).reshape(N, HV * nb, _DIM, K)
            return _pad_last(s, nb * _DIM).reshape(N, HV, K, nb, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV * nb, K, _DIM)
        h2, d2 = split(initial_state), split(dht)
        dq, dk, dv2, db2, dg2, dh2 = chunk_gated_delta_rule_bwd(
            q, k, v2, g2, beta.repeat_interleave(nb, dim=2), scale, h2, do2, d2, state_v_first,
            cu_seqlens, cu_seqlens_cpu, chunk_indices, chunk_size, q_rstd, k_rstd)
        # (dq, dk come back per q/k head: already summed over the value heads)
        dv = dv2.reshape(B, T, HV, nb * _DIM)[..., :V]
        db, dg = db2.reshape(B, T, HV, nb).sum(-1), dg2.reshape(B, T, HV, nb).sum(-1)
        dh0 = None
        if dh2 is not None:
            if state_v_first:
                dh0 = dh2.reshape(N, HV, nb * _DIM, K)[:, :, :V]
            else:
                dh0 = dh2.reshape(N, HV, nb, K, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV, K, nb * _DIM)[..., :V]
            dh0 = dh0.contiguous()
        return dq, dk, dv.contiguous(), db, dg, dh0

    out_dtype = q.dtype
    work = q.dtype if q.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    qw, kw = (aligned16(_pad_last(x.to(work), KD).contiguous()) for x in (q, k))
    vw, dow = (aligned16(_pad_last(x.to(work), _DIM).contiguous()) for x in (v, do))
    gw = None if g is None else as_f32(g).contiguous()
    bw = as_f32(beta).contiguous()

    def state_in(s):
        if s is None:
            return None
        want = (N, HV, V, K) if state_v_first else (N, HV, K, V)
        if tuple(s.shape) != want:
            raise ValueError(f'initial_state and dht must have shape {want}, got {tuple(s.shape)}')
        s = as_f32(s)
        if state_v_first:
            s = s.transpose(-1, -2)
        return aligned16(pad_last_two(s, KD, _DIM).contiguous())
    h0, dhtw = state_in(initial_state), state_in(dht)

    # FLA_HIP_BWD_SCAN_MODE forces one form of the two scans (default: automatic): whole sequences ('wide') or time segments
    # wherever they are possible at all ('segments')
    flags = {'wide': _lib.FLAG_SCAN_WIDE, 'segments': _lib.FLAG_SCAN_SEGMENTS}.get(os.environ.get('FLA_HIP_BWD_SCAN_MODE', 'auto'), 0)
    chunk_table = chunk_offsets = None
    if cu_seqlens is not None:
        if cu_seqlens.dtype not in (torch.int32, torch.int64):
            cu_seqlens = cu_seqlens.long()
        cu_seqlens = cu_seqlens.to(dev)
        if cu_seqlens.dtype == torch.int32:
            flags |= _lib.FLAG_CU_INT32
        check_cu_seqlens(cu_seqlens, T, cu_seqlens_cpu)
        chunk_indices = prepare_chunk_indices(cu_seqlens, _CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)      # (derived here, never taken over)
        chunk_table = chunk_indices.to(device=dev, dtype=cu_seqlens.dtype).contiguous()
        chunk_offsets = prepare_scan_tables(cu_seqlens, _CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)
        num_chunks = chunk_table.shape[0]
    else:
        num_chunks = B * ((T + _CHUNK - 1) // _CHUNK)

    # The kernels write the tokens inside [cu_seqlens[0], cu_seqlens[-1]) only.  Tokens of a packed tensor outside every
    # sequence get zero gradients (what autograd hands on, e.g. to a projection's weight gradient, must not be
    # uninitialised memory); the boundaries are known from the host summary that check_cu_seqlens has just memoised.
    alloc = torch.empty
    if cu_seqlens is not None:
        first, last = cu_bounds(cu_seqlens, cu_seqlens_cpu)
        if first != 0 or last != T:
            alloc = torch.zeros
    dq = alloc(B, T, HV, KD, dtype=work, device=dev)
    dk = alloc(B, T, HV, KD, dtype=work, device=dev)
    dv = alloc(B, T, HV, _DIM, dtype=work, device=dev)
    dg = alloc(B, T, HV, dtype=torch.float32, device=dev)
    db = alloc(B, T, HV, dtype=torch.float32, device=dev)
    dh0 = torch.empty(N, HV, KD, _DIM, dtype=torch.float32, device=dev) if initial_state is not None else None
    lib = _lib.load()
    ws_bytes = lib.gdn_chunk_bwd_qk_l2norm_workspace_bytes(num_chunks, HV, KD, B * T) if inside else lib.gdn_chunk_bwd_workspace_bytes(num_chunks, HV, KD)
    workspace = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    tail = (ptr(vw), ptr(gw), ptr(bw), ptr(h0), ptr(dow), ptr(dhtw),
            ptr(dq), ptr(dk), ptr(dv), ptr(dg), ptr(db), ptr(dh0),
            ptr(cu_seqlens), ptr(chunk_table), ptr(chunk_offsets), ptr(workspace), ws_bytes,
            B, T, H, HV, KD, _DIM, N, num_chunks, float(scale), dtype_code(work), _lib.DTYPE_F32, flags,
            current_stream_ptr(dev))
    _lib.check((lib.gdn_chunk_bwd_qk_l2norm if inside else lib.gdn_chunk_bwd)(ptr(qw), ptr(kw), *tail))
    dq = _finish(lib, dq, qw, q_rstd, H, K, out_dtype)
    dk = _finish(lib, dk, kw, k_rstd, H, K, out_dtype)
    dv = dv[..., :V].to(out_dtype)
    if dh0 is not None:
        dh0 = dh0[..., :K, :V]
        dh0 = (dh0.transpose(-1, -2) if state_v_first else dh0).contiguous()
    return dq, dk, dv, db, dg, dh0


def _finish(lib, dxh: torch.Tensor, y: torch.Tensor, rstd: torch.Tensor | None, H: int, K: int, out_dtype) -> torch.Tensor:
    """dq or dk per value head ``[B,T,HV,KD]`` -> per q/k head ``[B,T,H,K]``: the sum over the value heads of a
    q/k head and, with ``rstd``, the way back through the l2 normalisation (``y``: the normalised rows, KD wide)."""
    B, T, HV, D = dxh.shape
    if rstd is None and HV == H and K == D:
        return dxh.to(out_dtype)
    dx = torch.empty(B, T, H, K, dtype=dxh.dtype, device=dxh.device)
    if K % 8:                                       # (rows of the kernel are multiples of 8 elements)
        KP = (K + 7) // 8 * 8
        dx = torch.empty(B, T, H, KP, dtype=dxh.dtype, device=dxh.device)
    _lib.check(lib.gdn_l2norm_bwd(ptr(dxh), ptr(y) if rstd is not None else None, ptr(rstd), ptr(dx), B * T * H, HV // H, D,
                                  dx.shape[-1], dtype_code(dxh.dtype), current_stream_ptr(dxh.device)))
    return dx[..., :K].to(out_dtype)


def l2norm_fwd(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Rows divided by sqrt(sum x^2 + 1e-6), in x's dtype (fp32 input: bf16), and the factors ``[..., 1]`` fp32
    (fla/modules/l2norm.py:222-262).  Rows whose length is not a multiple of 8 come back zero-padded to one."""
    require_gpu(x)
    work = x.dtype if x.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    if x.shape[-1] > 256:
        raise NotImplementedError('l2norm_fwd: rows of up to 256 elements')
    x = _pad_last(x, (x.shape[-1] + 7) // 8 * 8)
    D = x.shape[-1]
    xw = aligned16(x.to(work).contiguous())
    y = torch.empty_like(xw)
    rstd = torch.empty(*x.shape[:-1], 1, dtype=torch.float32, device=x.device)
    _lib.check(_lib.load().gdn_l2norm_fwd(ptr(xw), ptr(y), ptr(rstd), xw.numel() // D, D, D, dtype_code(work),
                                          current_stream_ptr(x.device)))
    return y, rstd


class ChunkGatedDeltaRuleFunction(torch.autograd.Function):
    """Forward through the fused inference kernels, backward through ``gdn_chunk_bwd``."""

    @staticmethod
    def forward(ctx, q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first, cu_seqlens,
                cu_seqlens_cpu, chunk_indices, use_qk_l2norm_in_kernel, use_gate_in_kernel, A_log, dt_bias,
                use_beta_sigmoid_in_kernel, allow_neg_eigval, chunk_size):
        from fla_hip.ops.gated_delta_rule.chunk import chunk_gated_delta_rule_fwd
        o, ht = chunk_gated_delta_rule_fwd(
            q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first, cu_seqlens, cu_seqlens_cpu,
            chunk_indices, chunk_size, A_log if use_gate_in_kernel else None, dt_bias if use_gate_in_kernel else None,
            use_qk_l2norm_in_kernel, use_beta_sigmoid_in_kernel, allow_neg_eigval)
        ctx.save_for_backward(q, k, v, g, beta, initial_state, cu_seqlens, cu_seqlens_cpu, chunk_indices, A_log, dt_bias)
        ctx.opts = (scale, state_v_first, use_qk_l2norm_in_kernel, use_gate_in_kernel, use_beta_sigmoid_in_kernel,
                    allow_neg_eigval, chunk_size)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        q, k, v, g, beta_raw, h0, cu_seqlens, cu_seqlens_cpu, chunk_indices, A_log, dt_bias = ctx.saved_tensors
        scale, state_v_first, l2, gate, bsig, neg, chunk_size = ctx.opts
        K = q.shape[-1]
        beta = beta_raw
        if bsig:
            beta = torch.sigmoid(beta_raw.float()) * (2.0 if neg else 1.0)
        g_in = g
        if gate:
            # g = -exp(A_log) softplus(g + dt_bias)   (fla/ops/gated_delta_rule/gate.py:21-46)
            x = g_in.float() if dt_bias is None else g_in.float() + dt_bias.float()
            g = -A_log.float().exp() * F.softplus(x)
        dq, dk, dv, db, dg, dh0 = chunk_gated_delta_rule_bwd(
            q, k, v, g, beta, scale, h0, do.contiguous(), dht, state_v_first, cu_seqlens, cu_seqlens_cpu,
            chunk_indices, chunk_size, qk_l2norm=l2)
        if bsig:
            s = torch.sigmoid(beta_raw.float())
            db = db * s * (1 - s) * (2.0 if neg else 1.0)
        dA_log = ddt_bias = None
        if gate:
            # (gate.py:109-160)  dg/dx = -exp(A_log) sigmoid(x),  dg/dA_log = g
            dA_log = (dg * g).sum((0, 1)).to(A_log.dtype).reshape(A_log.shape)
            dg = dg * (-A_log.float().exp() * torch.sigmoid(x))
            if dt_bias is not None:
                ddt_bias = dg.sum((0, 1)).to(dt_bias.dtype).reshape(dt_bias.shape)
        if g_in is not None:
            dg = dg.to(g_in.dtype)
        else:
            dg = None
        return (dq[..., :K].to(q.dtype), dk[..., :K].to(k.dtype), dv.to(v.dtype), dg, db.to(beta_raw.dtype), None, dh0, None, None, None,
                None, None, None, None, dA_log, ddt_bias, None, None, None)
