"""``chunk_kda``: chunked prefill of the KDA operator (the gated delta rule with a decay per key feature), with the
signature, validation and error types of fla/ops/kda/chunk.py:178-443.  The reference's forward launches
(gate activation + chunk-local cumsum, the intra-chunk stage, ``recompute_w_u_fwd``, the state recurrence and the output,
fla/ops/kda/chunk_fwd.py:20-134) are one call into libgdn_hip.so (``gdn_chunk_kda_fwd``): a chunk-parallel kernel and a
sequential one.  The activations the reference fuses (l2 norm of q and k, gate, beta sigmoid) happen inside the first.
Its backward (``chunk_kda_bwd``, fla/ops/kda/chunk_bwd.py, behind ``ChunkKDAFunction``, chunk.py:23-175) is one call as well
(``gdn_chunk_kda_bwd``); nothing is kept from the forward call but its inputs, and the activations' derivatives are
elementwise work around that call."""
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


def chunk_kda_fwd(q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first=False, cu_seqlens=None,
                  cu_seqlens_cpu=None, A_log=None, dt_bias=None, lower_bound=None, gate_mode=0,
                  use_qk_l2norm_in_kernel=False, use_beta_sigmoid_in_kernel=False, allow_neg_eigval=False, return_states=False):
    """Returns ``(o [B,T,HV,V] in q's dtype, final_state fp32 or None)``; ``gate_mode`` 0: g is the log decay,
    1: ``-exp(A_log) softplus(g + dt_bias)``, 2: ``lower_bound sigmoid(exp(A_log) (g + dt_bias))``.  With ``return_states``
    a third result: the state in front of every chunk, ``[B, NT, HV, K, V]`` (``[1, chunks of all sequences, ...]`` for packed
    input; ``[..., V, K]`` with ``state_v_first``) in the kernels' operand dtype."""
    dev = require_gpu(q, k, v, g, beta)
    check_operand_shapes(q, k, v, beta=beta, gk=g)
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if K > _DIM:
        # Wide keys (the reference takes K up to 256, fla/ops/kda/chunk.py:409): the chunked kernels hold one block of 128 key
        # features, so the forward goes token by token on the recurrence kernel, which holds two - the same mathematics and the
        # same options, far slower on long prompts.  No states in front of the chunks (there are no chunks) and no backward.
        if K > 2 * _DIM or return_states:
            raise NotImplementedError(f'chunk_kda with key head dims above {_DIM}: forward only, without intermediate states, '
                                      f'up to {2 * _DIM} (got K={K}, return_intermediate_states={return_states})')
        from fla_hip.ops.gated_delta_rule.fused_recurrent import fused_recurrent_gated_delta_rule_fwd
        o, ht = fused_recurrent_gated_delta_rule_fwd(
            q, k, v, None, g, None, beta, A_log, dt_bias, scale, initial_state, output_final_state,
            use_qk_l2norm_in_kernel, use_beta_sigmoid_in_kernel, allow_neg_eigval, state_v_first, cu_seqlens,
            False, None, None, kda_gate_mode=gate_mode, lower_bound=0.0 if lower_bound is None else lower_bound)
        return o.to(q.dtype), ht
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    nb = (V + _DIM - 1) // _DIM
    if nb > 1:
        # value columns are independent: a head with V > 128 is nb heads of 128 columns that share q, k, g, beta
        v2 = _pad_last(v, nb * _DIM).reshape(B, T, HV * nb, _DIM)
        h2 = None
        if initial_state is not None:
            if state_v_first:
                h2 = F.pad(initial_state, (0, 0, 0, nb * _DIM - V)).reshape(N, HV * nb, _DIM, K)
            else:
                h2 = _pad_last(initial_state, nb * _DIM).reshape(N, HV, K, nb, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV * nb, K, _DIM)
        o2, ht2, *hs2 = chunk_kda_fwd(
            q, k, v2, g.repeat_interleave(nb, dim=2), beta.repeat_interleave(nb, dim=2), scale, h2, output_final_state,
            state_v_first, cu_seqlens, cu_seqlens_cpu, None if A_log is None else A_log.reshape(-1).repeat_interleave(nb),
            None if dt_bias is None else dt_bias.reshape(HV, K).repeat_interleave(nb, dim=0), lower_bound, gate_mode,
            use_qk_l2norm_in_kernel, use_beta_sigmoid_in_kernel, allow_neg_eigval, return_states)
        o = o2.reshape(B, T, HV, nb * _DIM)[..., :V].contiguous()
        ht = None
        if ht2 is not None:
            if state_v_first:
                ht = ht2.reshape(N, HV, nb * _DIM, K)[:, :, :V]
            else:
                ht = ht2.reshape(N, HV, nb, K, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV, K, nb * _DIM)[..., :V]
            ht = ht.contiguous()
        if return_states:
            hs = hs2[0]
            B1, NC = hs.shape[:2]
            if state_v_first:
                hs = hs.reshape(B1, NC, HV, nb * _DIM, K)[:, :, :, :V]
            else:
                hs = hs.reshape(B1, NC, HV, nb, K, _DIM).permute(0, 1, 2, 4, 3, 5).reshape(B1, NC, HV, K, nb * _DIM)[..., :V]
            return o, ht, hs.contiguous()
        return o, ht

    out_dtype = q.dtype
    work = q.dtype if q.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    qw, kw, vw = (aligned16(_pad_last(x.to(work), _DIM).contiguous()) for x in (q, k, v))
    gw = aligned16(_pad_last(as_f32(g), _DIM).contiguous())
    bw = as_f32(beta).contiguous()
    if A_log is not None:
        A_log = A_log.detach().to(device=dev, dtype=torch.float32).reshape(-1).contiguous()
        if A_log.numel() != HV:
            raise ValueError(f'A_log must have {HV} entries, got {A_log.numel()}')
    if dt_bias is not None:
        if dt_bias.numel() != HV * K:
            raise ValueError(f'dt_bias must have HV * K = {HV * K} elements, got {dt_bias.numel()}')
        dt_bias = _pad_last(dt_bias.detach().to(device=dev, dtype=torch.float32).reshape(HV, K), _DIM).contiguous()
    h0 = None
    if initial_state is not None:
        want = (N, HV, V, K) if state_v_first else (N, HV, K, V)
        if tuple(initial_state.shape) != want:
            raise ValueError(f'initial_state must have shape {want}, got {tuple(initial_state.shape)}')
        h0 = as_f32(initial_state)
        if state_v_first:
            h0 = h0.transpose(-1, -2)
        h0 = aligned16(pad_last_two(h0, _DIM, _DIM).contiguous())

    flags = 0
    if use_qk_l2norm_in_kernel:
        flags |= _lib.FLAG_QK_L2NORM
    if use_beta_sigmoid_in_kernel:
        flags |= _lib.FLAG_BETA_SIGMOID | (_lib.FLAG_NEG_EIGVAL if allow_neg_eigval else 0)
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
    hs = torch.empty(num_chunks, HV, _DIM, _DIM, dtype=work, device=dev) if return_states else None
    entry, states = (lib.gdn_chunk_kda_fwd_states, (ptr(hs),)) if return_states else (lib.gdn_chunk_kda_fwd, ())
    _lib.check(entry(
        ptr(qw), ptr(kw), ptr(vw), ptr(gw), ptr(bw), ptr(A_log), ptr(dt_bias),
        0.0 if lower_bound is None else float(lower_bound), gate_mode, ptr(h0), ptr(ht), ptr(o), *states,
        ptr(cu_seqlens), ptr(chunk_table), ptr(chunk_offsets), ptr(workspace), ws_bytes,
        B, T, H, HV, _DIM, _DIM, N, num_chunks, float(scale), dtype_code(work), _lib.DTYPE_F32, flags,
        current_stream_ptr(dev)))
    o = o[..., :V].to(out_dtype)
    if ht is not None:
        ht = ht[..., :K, :V]
        ht = (ht.transpose(-1, -2) if state_v_first else ht).contiguous()
    if return_states:
        hs = hs[..., :K, :V]
        hs = (hs.transpose(-1, -2) if state_v_first else hs).contiguous()
        return o, ht, hs.reshape(B if cu_seqlens is None else 1, -1, *hs.shape[1:]).to(out_dtype)
    return o, ht


def chunk_kda_bwd(q, k, v, g, beta, scale, initial_state, do, dht, state_v_first=False, cu_seqlens=None, cu_seqlens_cpu=None,
                  q_rstd=None, k_rstd=None):
    """q, k ``[B,T,H,K]``, v, do ``[B,T,HV,V]``, g ``[B,T,HV,K]`` (log decays), beta ``[B,T,HV]`` as the recurrence uses them.
    Returns ``(dq, dk, dv, dbeta, dg, dh0)``: dq, dk, dv in q's dtype, dbeta ``[B,T,HV]`` and dg ``[B,T,HV,K]`` fp32, dh0 fp32
    (None without ``initial_state``).  With ``q_rstd``, ``k_rstd`` (what ``l2norm_fwd`` returns next to the normalised rows
    passed as q and k) dq and dk are the gradients of the rows before normalisation."""
    dev = require_gpu(q, k, v, g, beta, do)
    check_operand_shapes(q, k, v, beta=beta, gk=g)
    if do.shape != v.shape:
        raise ValueError(f'do must have the shape of v, got {tuple(do.shape)} and {tuple(v.shape)}')
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if K > _DIM:
        raise NotImplementedError(f'the chunked KDA kernels cover key head dims up to {_DIM} (got K={K})')
    N = B if cu_seqlens is None else len(cu_seqlens) - 1
    nb = (V + _DIM - 1) // _DIM
    if nb > 1:
        # value columns are independent: a head with V > 128 is nb heads of 128 columns that share q, k, g, beta
        def split(s):       # [N, HV, K, V] -> [N, HV*nb, K, 128]  (V-first: [N, HV, V, K] -> [N, HV*nb, 128, K])
            if s is None:
                return None
            if state_v_first:
                return F.pad(s, (0, 0, 0, nb * _DIM - V)).reshape(N, HV * nb, _DIM, K)
            return _pad_last(s, nb * _DIM).reshape(N, HV, K, nb, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV * nb, K, _DIM)
        v2 = _pad_last(v, nb * _DIM).reshape(B, T, HV * nb, _DIM)
        do2 = _pad_last(do, nb * _DIM).reshape(B, T, HV * nb, _DIM)
        dq, dk, dv2, db2, dg2, dh2 = chunk_kda_bwd(
            q, k, v2, g.repeat_interleave(nb, dim=2), beta.repeat_interleave(nb, dim=2), scale, split(initial_state), do2,
            split(dht), state_v_first, cu_seqlens, cu_seqlens_cpu, q_rstd, k_rstd)
        dv = dv2.reshape(B, T, HV, nb * _DIM)[..., :V].contiguous()
        db, dg = db2.reshape(B, T, HV, nb).sum(-1), dg2.reshape(B, T, HV, nb, K).sum(-2)
        dh0 = None
        if dh2 is not None:
            if state_v_first:
                dh0 = dh2.reshape(N, HV, nb * _DIM, K)[:, :, :V]
            else:
                dh0 = dh2.reshape(N, HV, nb, K, _DIM).permute(0, 1, 3, 2, 4).reshape(N, HV, K, nb * _DIM)[..., :V]
            dh0 = dh0.contiguous()
        return dq, dk, dv, db, dg, dh0

    out_dtype = q.dtype
    work = q.dtype if q.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    qw, kw, vw, dow = (aligned16(_pad_last(x.to(work), _DIM).contiguous()) for x in (q, k, v, do))
    gw = aligned16(_pad_last(as_f32(g), _DIM).contiguous())
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
        return aligned16(pad_last_two(s, _DIM, _DIM).contiguous())
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

    dq, dk, dv = (alloc(B, T, HV, _DIM, dtype=work, device=dev) for _ in range(3))
    dg = alloc(B, T, HV, _DIM, dtype=torch.float32, device=dev)
    db = alloc(B, T, HV, dtype=torch.float32, device=dev)
    dh0 = torch.empty(N, HV, _DIM, _DIM, dtype=torch.float32, device=dev) if initial_state is not None else None
    lib = _lib.load()
    ws_bytes = lib.gdn_chunk_kda_bwd_workspace_bytes(num_chunks, HV)
    workspace = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
    _lib.check(lib.gdn_chunk_kda_bwd(
        ptr(qw), ptr(kw), ptr(vw), ptr(gw), ptr(bw), ptr(h0), ptr(dow), ptr(dhtw),
        ptr(dq), ptr(dk), ptr(dv), ptr(dg), ptr(db), ptr(dh0),
        ptr(cu_seqlens), ptr(chunk_table), ptr(chunk_offsets), ptr(workspace), ws_bytes,
        B, T, H, HV, _DIM, _DIM, N, num_chunks, float(scale), dtype_code(work), _lib.DTYPE_F32, flags,
        current_stream_ptr(dev)))
    dq = _finish(lib, dq, qw, q_rstd, H, K, out_dtype)
    dk = _finish(lib, dk, kw, k_rstd, H, K, out_dtype)
    dv = dv[..., :V].to(out_dtype)
    dg = dg[..., :K]
    if dh0 is not None:
        dh0 = dh0[..., :K, :V]
        dh0 = (dh0.transpose(-1, -2) if state_v_first else dh0).contiguous()
    return dq, dk, dv, db, dg, dh0


def _kda_gate(g, A_log, dt_bias, lower_bound):
    """The gate activation in fp32 (fla/ops/kda/gate.py:27-94) and what its derivative needs: returns
    ``(log decay, x = g + dt_bias, a = exp(A_log) per head or None)``."""
    HV, K = g.shape[-2:]
    x = g.float()
    if dt_bias is not None:
        x = x + dt_bias.float().reshape(HV, K)
    a = None if A_log is None else A_log.float().exp().reshape(HV, 1)
    if lower_bound is not None:
        return lower_bound * torch.sigmoid(x if a is None else a * x), x, a
    return -(a if a is not None else torch.e) * F.softplus(x), x, a


class ChunkKDAFunction(torch.autograd.Function):
    """Forward through ``gdn_chunk_kda_fwd``, backward through ``gdn_chunk_kda_bwd`` (fla/ops/kda/chunk.py:23-175)."""

    @staticmethod
    def forward(ctx, q, k, v, g, beta, A_log, dt_bias, scale, initial_state, output_final_state, use_qk_l2norm_in_kernel,
                gate_mode, use_beta_sigmoid_in_kernel, allow_neg_eigval, state_v_first, cu_seqlens, cu_seqlens_cpu, lower_bound):
        o, ht = chunk_kda_fwd(q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first, cu_seqlens,
                              cu_seqlens_cpu, A_log, dt_bias, lower_bound, gate_mode, use_qk_l2norm_in_kernel,
                              use_beta_sigmoid_in_kernel, allow_neg_eigval)
        ctx.save_for_backward(q, k, v, g, beta, A_log, dt_bias, initial_state, cu_seqlens, cu_seqlens_cpu)
        ctx.opts = (scale, use_qk_l2norm_in_kernel, gate_mode, use_beta_sigmoid_in_kernel, allow_neg_eigval, state_v_first, lower_bound)
        return o, ht

    @staticmethod
    def backward(ctx, do, dht):
        q, k, v, g_in, beta_raw, A_log, dt_bias, h0, cu_seqlens, cu_seqlens_cpu = ctx.saved_tensors
        scale, l2, gate_mode, bsig, neg, state_v_first, lower_bound = ctx.opts
        q_rstd = k_rstd = None
        qn, kn = q, k
        if l2:
            (qn, q_rstd), (kn, k_rstd) = l2norm_fwd(q), l2norm_fwd(k)
            qn, kn = qn[..., :q.shape[-1]], kn[..., :k.shape[-1]]       # (l2norm_fwd pads rows to a multiple of 8)
        beta = beta_raw
        if bsig:
            beta = torch.sigmoid(beta_raw.float()) * (2.0 if neg else 1.0)
        g = g_in
        if gate_mode:
            g, x, a = _kda_gate(g_in, A_log, dt_bias, lower_bound if gate_mode == 2 else None)
        dq, dk, dv, db, dg, dh0 = chunk_kda_bwd(qn, kn, v, g, beta, scale, h0, do.contiguous(), dht, state_v_first,
                                                cu_seqlens, cu_seqlens_cpu, q_rstd, k_rstd)
        if bsig:
            s = torch.sigmoid(beta_raw.float())
            db = db * s * (1 - s) * (2.0 if neg else 1.0)
        dA_log = ddt_bias = None
        if gate_mode:
            # (fla/ops/kda/gate.py)  softplus form: dg/dx = -a sigmoid(x), dg/dA_log = g;  bounded form, s = sigmoid(a x):
            # dg/dx = lower_bound s (1 - s) a, dg/dA_log = lower_bound s (1 - s) a x
            if gate_mode == 2:
                s = torch.sigmoid(x if a is None else a * x)
                ds = dg * (lower_bound * s * (1 - s))
                if A_log is not None:
                    dA_log = (ds * a * x).sum((0, 1, 3)).to(A_log.dtype).reshape(A_log.shape)
                    ds = ds * a
                dg = ds
            else:
                if A_log is not None:
                    dA_log = (dg * g).sum((0, 1, 3)).to(A_log.dtype).reshape(A_log.shape)
                dg = dg * (-(a if a is not None else torch.e) * torch.sigmoid(x))
            if dt_bias is not None:
                ddt_bias = dg.sum((0, 1)).to(dt_bias.dtype).reshape(dt_bias.shape)
        K = q.shape[-1]
        return (dq[..., :K].to(q.dtype), dk[..., :K].to(k.dtype), dv.to(v.dtype), dg.to(g_in.dtype), db.to(beta_raw.dtype), dA_log, ddt_bias,
                None, dh0, None, None, None, None, None, None, None, None, None)


@torch.compiler.disable
def chunk_kda(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    scale: float | None = None,
    initial_state: torch.Tensor | None = None,
    output_final_state: bool = False,
    use_qk_l2norm_in_kernel: bool = False,
    use_gate_in_kernel: bool = False,
    use_beta_sigmoid_in_kernel: bool = False,
    allow_neg_eigval: bool = False,
    safe_gate: bool = False,
    lower_bound: float | None = None,
    disable_recompute: bool = False,
    return_intermediate_states: bool = False,
    state_v_first: bool = False,
    cu_seqlens: torch.LongTensor | None = None,
    cu_seqlens_cpu: torch.LongTensor | None = None,
    cp_context=None,
    **kwargs,
):
    r"""Chunked KDA (prefill); differentiable in q, k, v, g, beta, ``A_log``, ``dt_bias`` and ``initial_state``.

    Args:
        q, k: ``[B, T, H, K]``; v: ``[B, T, HV, V]`` with ``HV % H == 0``.
        g: ``[B, T, HV, K]`` log decay per key feature, or the raw gate input with ``use_gate_in_kernel=True``
            (``A_log [HV]`` and optional ``dt_bias [HV * K]`` as keywords: ``-exp(A_log) softplus(g + dt_bias)``, or with
            ``lower_bound`` (``safe_gate``) ``lower_bound sigmoid(exp(A_log) (g + dt_bias))``).
        beta: ``[B, T, HV]`` (logits with ``use_beta_sigmoid_in_kernel``; ``allow_neg_eigval`` doubles the sigmoid).
        scale: defaults to ``K ** -0.5``.  initial_state: ``[N, HV, K, V]`` (``[N, HV, V, K]`` with ``state_v_first``).
        safe_gate: accepted; the kernels form the intra-chunk decays pair by pair inside blocks of 16 rows whatever the
            gate's range, so it changes nothing here.  disable_recompute: accepted; the backward pass always computes the
            forward's intermediates again.
        return_intermediate_states: in inference mode a third result, the state in front of every chunk
            ``[B, NT, HV, K, V]`` in q's dtype (fla/ops/kda/chunk.py:98-100).  cp_context: not part of this build.
        cu_seqlens: ``[N + 1]`` boundaries of packed sequences (then ``B == 1``).

    Returns:
        ``(o [B, T, HV, V] in q's dtype, final_state or None)``.
    """
    if cp_context is not None:
        raise NotImplementedError('context parallelism (cp_context) is outside this single-GPU build')
    if 'transpose_state_layout' in kwargs:
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
    H, HV = q.shape[2], v.shape[2]
    if q.shape[2] != k.shape[2] or HV % H != 0:
        raise ValueError(f'q and k must share their heads and HV={HV} must be a multiple of H={H}')
    if g.shape != (*v.shape[:3], k.shape[-1]):
        raise ValueError(f'g must have shape {(*v.shape[:3], k.shape[-1])}, got {tuple(g.shape)}')
    chunk_size = kwargs.pop('chunk_size', 64)
    if chunk_size not in (16, 32, 64):
        raise ValueError(f'`chunk_size` must be 16, 32, or 64, got {chunk_size}.')
    if allow_neg_eigval and not use_beta_sigmoid_in_kernel:
        raise ValueError('`allow_neg_eigval=True` requires `use_beta_sigmoid_in_kernel=True`.')
    if safe_gate and lower_bound is None:
        raise ValueError('`safe_gate=True` requires `lower_bound`.')
    A_log, dt_bias = kwargs.get('A_log'), kwargs.get('dt_bias')
    gate_mode = 0
    if use_gate_in_kernel:
        if A_log is None and lower_bound is None:
            raise AssertionError('A_log must be provided when use_gate_in_kernel=True (unless lower_bound is set).')
        gate_mode = 2 if lower_bound is not None else 1
    else:
        A_log = dt_bias = None
    if scale is None:
        scale = k.shape[-1] ** -0.5
    if return_intermediate_states:
        # (the reference's conditions, fla/ops/kda/chunk.py:98-100)
        assert torch.is_inference_mode_enabled(), 'return_intermediate_states is only allowed in inference mode'
        assert disable_recompute is False, 'return_intermediate_states must be used with disable_recompute=False'
        return chunk_kda_fwd(q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first, cu_seqlens,
                             cu_seqlens_cpu, A_log, dt_bias, lower_bound, gate_mode, use_qk_l2norm_in_kernel,
                             use_beta_sigmoid_in_kernel, allow_neg_eigval, return_states=True)
    if torch.is_grad_enabled() and any(x is not None and x.requires_grad for x in (q, k, v, g, beta, A_log, dt_bias, initial_state)):
        if k.shape[-1] > _DIM:
            raise NotImplementedError(f'chunk_kda with key head dims above {_DIM} is forward only (got K={k.shape[-1]})')
        return ChunkKDAFunction.apply(q, k, v, g, beta, A_log, dt_bias, scale, initial_state, output_final_state,
                                      use_qk_l2norm_in_kernel, gate_mode, use_beta_sigmoid_in_kernel, allow_neg_eigval,
                                      state_v_first, cu_seqlens, cu_seqlens_cpu, lower_bound)
    return chunk_kda_fwd(q, k, v, g, beta, scale, initial_state, output_final_state, state_v_first, cu_seqlens,
                         cu_seqlens_cpu, A_log, dt_bias, lower_bound, gate_mode, use_qk_l2norm_in_kernel,
                         use_beta_sigmoid_in_kernel, allow_neg_eigval)
