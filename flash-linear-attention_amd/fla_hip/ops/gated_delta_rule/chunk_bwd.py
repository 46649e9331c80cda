"""Backward of ``chunk_gated_delta_rule``: ``chunk_gated_delta_rule_bwd`` with the argument meaning of
fla/ops/gated_delta_rule/chunk.py:125-257 and the autograd function around forward and backward
(chunk.py:260-395).  One call into libgdn_hip.so (``gdn_chunk_bwd``) replaces the reference's seven launches;
nothing is kept from the forward call but its inputs (A, w, u, the per-chunk states and v_new are computed
again).  The activations the forward kernels apply themselves (l2 norm of q and k, gate, beta sigmoid) and
their derivatives are elementwise work around that call, as in the reference (chunk.py:278-288, 385-393)."""
from __future__ import annotations

import torch
import torch.nn.functional as F

from fla_hip import _lib
from fla_hip.ops.gated_delta_rule._common import aligned16, as_f32, current_stream_ptr, dtype_code, ptr, require_gpu
from fla_hip.ops.utils.index import prepare_chunk_indices, prepare_scan_tables

_CHUNK = 64
_DIM = 128          # head dims of the backward kernels; smaller ones are zero-padded


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
):
    """q, k ``[B,T,H,K]``, v, do ``[B,T,HV,V]``, g (log decay), beta ``[B,T,HV]`` as the recurrence uses them.
    Returns ``(dq, dk, dv, dbeta, dg, dh0)``: dq, dk, dv in q's dtype, dbeta, dg fp32, dh0 fp32 (None without
    ``initial_state``)."""
    dev = require_gpu(q, k, v, beta, do)
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if K > _DIM:
        raise NotImplementedError(f'the backward kernels cover head dims up to {_DIM} (got K={K})')
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
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
            cu_seqlens, cu_seqlens_cpu, chunk_indices, chunk_size)
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
    qw, kw = (aligned16(_pad_last(x.to(work), _DIM).contiguous()) for x in (q, k))
    vw, dow = (aligned16(_pad_last(x.to(work), _DIM).contiguous()) for x in (v, do))
    gw = None if g is None else as_f32(g).contiguous()
    bw = as_f32(beta).contiguous()

    def state_in(s):
        if s is None:
            return None
        s = as_f32(s)
        if state_v_first:
            s = s.transpose(-1, -2)
        return aligned16(F.pad(s, (0, _DIM - V, 0, _DIM - K)).contiguous())
    h0, dhtw = state_in(initial_state), state_in(dht)

    flags = 0
    chunk_table = chunk_offsets = None
    if cu_seqlens is not None:
        if cu_seqlens.dtype not in (torch.int32, torch.int64):
            cu_seqlens = cu_seqlens.long()
        cu_seqlens = cu_seqlens.to(dev)
        if cu_seqlens.dtype == torch.int32:
            flags |= _lib.FLAG_CU_INT32
        if chunk_indices is None or chunk_size != _CHUNK:
            chunk_indices = prepare_chunk_indices(cu_seqlens, _CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)
        chunk_table = chunk_indices.to(device=dev, dtype=cu_seqlens.dtype).contiguous()
        chunk_offsets = prepare_scan_tables(cu_seqlens, _CHUNK, cu_seqlens_cpu=cu_seqlens_cpu)
        num_chunks = chunk_table.shape[0]
    else:
        num_chunks = B * ((T + _CHUNK - 1) // _CHUNK)

    # rows past a sequence's end inside its last chunk are never written: start from zeros only where that matters
    dq = torch.empty(B, T, HV, _DIM, dtype=work, device=dev)
    dk = torch.empty(B, T, HV, _DIM, dtype=work, device=dev)
    dv = torch.empty(B, T, HV, _DIM, dtype=work, device=dev)
    dg = torch.empty(B, T, HV, dtype=torch.float32, device=dev)
    db = torch.empty(B, T, HV, dtype=torch.float32, device=dev)
    dh0 = torch.empty(N, HV, _DIM, _DIM, dtype=torch.float32, device=dev) if initial_state is not None else None
    lib = _lib.load()
    ws_bytes = lib.gdn_chunk_bwd_workspace_bytes(num_chunks, HV)
    workspace = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    _lib.check(lib.gdn_chunk_bwd(
        ptr(qw), ptr(kw), ptr(vw), ptr(gw), ptr(bw), ptr(h0), ptr(dow), ptr(dhtw),
        ptr(dq), ptr(dk), ptr(dv), ptr(dg), ptr(db), ptr(dh0),
        ptr(cu_seqlens), ptr(chunk_table), ptr(chunk_offsets), ptr(workspace), ws_bytes,
        B, T, H, HV, _DIM, _DIM, N, num_chunks, float(scale), dtype_code(work), _lib.DTYPE_F32, flags,
        current_stream_ptr(dev)))
    if HV != H:
        # grouped value heads: a q/k head collects the gradients of its HV/H value heads
        dq = dq.view(B, T, H, HV // H, _DIM).float().sum(3)
        dk = dk.view(B, T, H, HV // H, _DIM).float().sum(3)
    dq, dk, dv = dq[..., :K].to(out_dtype), dk[..., :K].to(out_dtype), dv[..., :V].to(out_dtype)
    if dh0 is not None:
        dh0 = dh0[..., :K, :V]
        dh0 = (dh0.transpose(-1, -2) if state_v_first else dh0).contiguous()
    return dq, dk, dv, db, dg, dh0


def _l2norm(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """rows divided by sqrt(sum x^2 + 1e-6), in x's dtype, and the factors (fla/modules/l2norm.py:84-109)"""
    xf = x.float()
    rstd = torch.rsqrt(xf.square().sum(-1, keepdim=True) + 1e-6)
    return (xf * rstd).to(x.dtype), rstd


def _l2norm_bwd(y: torch.Tensor, rstd: torch.Tensor, dy: torch.Tensor) -> torch.Tensor:
    """(fla/modules/l2norm.py:112-146)  dx = (dy - y <dy, y>) * rstd"""
    yf, dyf = y.float(), dy.float()
    return (dyf - yf * (dyf * yf).sum(-1, keepdim=True)) * rstd


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
        q_rstd = k_rstd = None
        if l2:
            q, q_rstd = _l2norm(q)
            k, k_rstd = _l2norm(k)
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
            chunk_indices, chunk_size)
        if l2:
            dq = _l2norm_bwd(q, q_rstd, dq)
            dk = _l2norm_bwd(k, k_rstd, dk)
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
        return (dq.to(q.dtype), dk.to(k.dtype), dv.to(v.dtype), dg, db.to(beta_raw.dtype), None, dh0, None, None, None,
                None, None, None, None, dA_log, ddt_bias, None, None, None)
