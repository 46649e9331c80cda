"""CPU oracle for the gated delta rule (Gated DeltaNet) inference path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
module: it is the checker used by ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py``.  It is a restatement, in plain torch
CPU ops, of the algorithm in the reference's files (paths relative to the
reference checkout):

* ``fla/ops/gated_delta_rule/naive.py:13-64``    token recurrence
* ``fla/ops/gated_delta_rule/naive.py:67-161``   chunked form
* ``fla/ops/gated_delta_rule/chunk.py:33-123``   stage order of the chunk pipeline
* ``fla/ops/utils/cumsum.py:33-68``              chunk-local gate cumsum
* ``fla/ops/gated_delta_rule/chunk_fwd.py:137-291``  gated beta*K*K^T and its unit-lower inverse
* ``fla/ops/gated_delta_rule/wy_fast.py:72-106`` WY factors w, u
* ``fla/ops/common/chunk_delta_h.py:174-348``    inter-chunk state recurrence
* ``fla/ops/common/chunk_o.py:94-153``           output
* ``fla/ops/gated_delta_rule/fused_recurrent.py:66-181``  decode recurrence and its flags
* ``fla/ops/utils/index.py:113-172``             varlen chunk tables
* ``fla/modules/l2norm.py:84-109``, ``fla/ops/gated_delta_rule/gate.py:21-46``  prologues
* ``fla/utils/_testing.py:19-41``                error metric
* ``fla/ops/kda/naive.py:12-66``, ``fla/ops/kda/gate.py:27-94``, ``fla/ops/kda/fused_recurrent.py:150-181``
  the KDA operator's token recurrence (a decay per key feature) and its gate activations
* ``fla/ops/comba/fused_recurrent.py:85-105``, ``fla/ops/comba/naive.py:70-171``  the comba operator (a second key for the
  prediction, made before the token's decay): token recurrence and chunked form
* ``fla/ops/gated_delta_rule/chunk.py:125-257``, ``fla/ops/common/chunk_delta_h.py:369-560``, ``fla/ops/common/chunk_o.py:172-357``,
  ``fla/ops/gated_delta_rule/wy_fast.py:123-296``  the chunked backward pass, stage by stage (``chunk_backward_one_sequence``);
  the gradients themselves are reverse-mode differentiation of the token recurrence (``gated_delta_rule_grads``)

Parity pins (all in ``tests/test_oracle.py``): scalar brute force written as
independent pure-python loops on tiny shapes, closed forms for one decode step
(beta=0, exact projection), ``torch.linalg.inv`` for the triangular solve,
recurrent == chunked, split-in-time hand-off, varlen == per-sequence loop,
GVA == repeat_interleave, state_v_first == transpose, and the committed
fixtures under ``tests/golden/`` (a second set of scalar fixtures pins the
optional arguments gk, gv, beta per value column and the pooled states of
speculative decoding).  The KDA recurrence is the gk branch of the token recurrence (pinned by those
fixtures); its gate activations are pinned by values that the formulas fix (``test_kda_gate_pins``).
The gradients (``gated_delta_rule_grads``) are pinned by central finite differences of the recurrence in fp64 for every input
and every prologue, and the stage-by-stage backward agrees with them to 1e-12 (``tests/test_chunk_bwd.py``).
The comba recurrence is pinned by scalar loops, by its chunked form (library triangular solve) and by its reduction to the
delta rule at p = k, g = 0 (``test_comba_*`` in ``tests/test_oracle.py``).  Its gradients (``comba_grads``) and those of the KDA recurrence
(``kda_grads``, every gate activation) are pinned by central finite
differences of that recurrence in fp64 for every input (``test_comba_grads_match_finite_differences``).
No function here is "parity unpinned".

Everything is computed in ``dtype`` (float32 by default, float64 for tight
pins); inputs are upcast first, so bf16 inputs are consumed as their exact
rounded values.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F

RCP_LN2 = 1.4426950216  # fla/ops/utils/constant.py:10


# --------------------------------------------------------------------------- #
# error metric (fla/utils/_testing.py:19-26)
# --------------------------------------------------------------------------- #
def get_abs_err(x: torch.Tensor, y: torch.Tensor) -> float:
    return (x.detach().double() - y.detach().double()).flatten().abs().max().item()


def get_err_ratio(x: torch.Tensor, y: torch.Tensor) -> float:
    x, y = x.detach().double(), y.detach().double()
    err = (x - y).flatten().square().mean().sqrt().item()
    base = x.flatten().square().mean().sqrt().item()
    return err / (base + 1e-8)


def max_abs_ratio(ref: torch.Tensor, x: torch.Tensor) -> float:
    """max|ref - x| / max|ref|, the second tolerance the build is held to."""
    ref, x = ref.detach().double(), x.detach().double()
    return (ref - x).abs().max().item() / (ref.abs().max().item() + 1e-12)


# --------------------------------------------------------------------------- #
# prologues
# --------------------------------------------------------------------------- #
def l2norm(x: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """x / sqrt(sum(x^2) + eps) over the last dim (fla/modules/l2norm.py:105-106)."""
    xf = x.to(torch.float64 if x.dtype == torch.float64 else torch.float32)
    return xf / torch.sqrt((xf * xf).sum(-1, keepdim=True) + eps)


def gdn_gate(g: torch.Tensor, A_log: torch.Tensor, dt_bias: torch.Tensor | None = None) -> torch.Tensor:
    """g = -exp(A_log) * softplus(g + dt_bias) (fla/ops/gated_delta_rule/gate.py:21-46)."""
    dt = torch.float64 if g.dtype == torch.float64 else torch.float32
    g = g.to(dt)
    if dt_bias is not None:
        g = g + dt_bias.to(dt)
    return -A_log.to(dt).exp() * F.softplus(g)


def kda_gate(g: torch.Tensor, A_log: torch.Tensor | None = None, dt_bias: torch.Tensor | None = None,
             lower_bound: float | None = None) -> torch.Tensor:
    """Log decay per key feature from the raw gate g [..., HV, K] (fla/ops/kda/gate.py:27-94): with a bias
    dt_bias [HV * K] added first, ``-exp(A_log[hv]) * softplus(g)``, or with a lower bound
    ``lower_bound * sigmoid(exp(A_log[hv]) * g)``.  Without A_log the factor is 1 under the sigmoid and exp(1) in
    front of the softplus (the recurrent kernel's constant, fla/ops/kda/fused_recurrent.py:168-181)."""
    HV, K = g.shape[-2:]
    dt = torch.float64 if g.dtype == torch.float64 else torch.float32       # (fp64 for the finite-difference pins)
    x = g.to(dt)
    if dt_bias is not None:
        x = x + dt_bias.to(dt).reshape(HV, K)
    if lower_bound is not None:
        if A_log is not None:
            x = x * A_log.to(dt).exp().reshape(HV, 1)
        return lower_bound * torch.sigmoid(x)
    a = A_log.to(dt).exp().reshape(HV, 1) if A_log is not None else math.e
    return -a * F.softplus(x)


# --------------------------------------------------------------------------- #
# varlen chunk tables (fla/ops/utils/index.py:113-172), as plain loops
# --------------------------------------------------------------------------- #
def prepare_lens(cu_seqlens) -> list[int]:
    cu = [int(x) for x in cu_seqlens]
    return [b - a for a, b in zip(cu[:-1], cu[1:])]


def prepare_chunk_indices(cu_seqlens, chunk_size: int) -> list[list[int]]:
    """[[sequence id, chunk id inside that sequence], ...] in packed order."""
    out = []
    for n, L in enumerate(prepare_lens(cu_seqlens)):
        for c in range((L + chunk_size - 1) // chunk_size):
            out.append([n, c])
    return out


def prepare_chunk_offsets(cu_seqlens, chunk_size: int) -> list[int]:
    """Exclusive prefix sum of per-sequence chunk counts, length N+1."""
    out = [0]
    for L in prepare_lens(cu_seqlens):
        out.append(out[-1] + (L + chunk_size - 1) // chunk_size)
    return out


# --------------------------------------------------------------------------- #
# token recurrence (naive.py:13-64 generalised to GVA / varlen / flags of
# fused_recurrent.py:114-174)
# --------------------------------------------------------------------------- #
def _expand_heads(x: torch.Tensor, HV: int) -> torch.Tensor:
    """GVA: q/k head h serves v heads h*G .. h*G+G-1 (i_h = i_hv // (HV // H),
    fused_recurrent.py:69); same as repeat_interleave on the head dim."""
    H = x.shape[2]
    if H == HV:
        return x
    return x.repeat_interleave(HV // H, dim=2)


def recurrent_gated_delta_rule(
    q, k, v, g=None, beta=None, scale=None, initial_state=None, output_final_state=False,
    cu_seqlens=None, gk=None, gv=None,
    use_qk_l2norm_in_kernel=False, use_gate_in_kernel=False, A_log=None, dt_bias=None,
    use_beta_sigmoid_in_kernel=False, allow_neg_eigval=False, state_v_first=False,
    dtype=torch.float32,
):
    """Per token:  S *= exp(g);  v' = beta*(v - S^T k);  S += k v'^T;  o = S^T (q*scale).

    q, k: [B,T,H,K]; v: [B,T,HV,V]; g, beta: [B,T,HV] (beta may be [B,T,HV,V]);
    initial_state: [N,HV,K,V] ([N,HV,V,K] if state_v_first).  With cu_seqlens B
    must be 1 and sequences are the packed slices.  Returns (o [B,T,HV,V] in
    ``dtype``, final_state [N,HV,K,V] in ``dtype`` or None).
    """
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if scale is None:
        scale = K ** -0.5
    qf, kf, vf = q.to(dtype), k.to(dtype), v.to(dtype)
    if use_qk_l2norm_in_kernel:
        qf = qf / torch.sqrt((qf * qf).sum(-1, keepdim=True) + 1e-6)
        kf = kf / torch.sqrt((kf * kf).sum(-1, keepdim=True) + 1e-6)
    qf, kf = _expand_heads(qf, HV), _expand_heads(kf, HV)
    if beta is None:
        bf = torch.ones(B, T, HV, dtype=dtype)
    else:
        bf = beta.to(dtype)
        if use_beta_sigmoid_in_kernel:
            bf = torch.sigmoid(bf) * (2.0 if allow_neg_eigval else 1.0)
    if bf.dim() == 3:
        bf = bf[..., None]                      # headwise beta broadcasts over V
    gf = None
    if g is not None:
        gf = gdn_gate(g, A_log, dt_bias).to(dtype) if use_gate_in_kernel else g.to(dtype)
    gkf = gk.to(dtype) if gk is not None else None
    gvf = gv.to(dtype) if gv is not None else None

    if cu_seqlens is None:
        bounds = [(b, 0, T) for b in range(B)]
    else:
        cu = [int(x) for x in cu_seqlens]
        bounds = [(0, s, e) for s, e in zip(cu[:-1], cu[1:])]
    N = len(bounds)
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    ht = torch.zeros(N, HV, K, V, dtype=dtype)
    for n, (b, s, e) in enumerate(bounds):
        S = torch.zeros(HV, K, V, dtype=dtype)
        if initial_state is not None:
            S0 = initial_state[n].to(dtype)
            S = S0.transpose(-1, -2).clone() if state_v_first else S0.clone()
        for t in range(s, e):
            if gf is not None:
                S = S * gf[b, t].exp()[:, None, None]
            if gkf is not None:
                S = S * gkf[b, t].exp()[:, :, None]
            if gvf is not None:
                S = S * gvf[b, t].exp()[:, None, :]
            kt, qt = kf[b, t], qf[b, t]                          # [HV,K]
            vp = bf[b, t] * (vf[b, t] - torch.einsum('hkv,hk->hv', S, kt))
            S = S + kt[:, :, None] * vp[:, None, :]
            o[b, t] = torch.einsum('hkv,hk->hv', S, qt * scale)
        ht[n] = S
    if not output_final_state:
        return o, None
    return o, (ht.transpose(-1, -2).contiguous() if state_v_first else ht)


def recurrent_kda(
    q, k, v, g, beta, scale=None, initial_state=None, output_final_state=False, cu_seqlens=None,
    use_qk_l2norm_in_kernel=False, use_gate_in_kernel=False, A_log=None, dt_bias=None, lower_bound=None,
    use_beta_sigmoid_in_kernel=False, allow_neg_eigval=False, state_v_first=False, dtype=torch.float32,
):
    """Token recurrence of the KDA operator (fla/ops/kda/naive.py:12-66): per token S *= exp(g)[:, None] with
    g [B,T,HV,K] a decay per key feature, then the delta-rule update and the read-out of the gated delta rule.
    With use_gate_in_kernel g is the raw gate (kda_gate)."""
    gk = kda_gate(g, A_log, dt_bias, lower_bound) if use_gate_in_kernel else g
    return recurrent_gated_delta_rule(
        q, k, v, None, beta, scale, initial_state, output_final_state, cu_seqlens, gk=gk,
        use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, use_beta_sigmoid_in_kernel=use_beta_sigmoid_in_kernel,
        allow_neg_eigval=allow_neg_eigval, state_v_first=state_v_first, dtype=dtype)


def recurrent_comba(
    q, k, v, p, g, beta=None, scale=None, initial_state=None, output_final_state=False, cu_seqlens=None,
    use_qk_l2norm_in_kernel=False, dtype=torch.float32,
):
    """Token recurrence of the comba operator as its kernels run it (fla/ops/comba/fused_recurrent.py:85-105; the chunked
    form fla/ops/comba/naive.py:70-171, which the reference's tests take as the truth, is the same map): the prediction
    uses a second key p and the state BEFORE this token's decay,
        v' = beta (v - S^T p);  S <- e^g S + k v'^T;  o = S^T (q scale).
    q, k, p: [B,T,H,K]; v: [B,T,HV,V]; g: [B,T,HV]; beta: [B,T,HV] or, one per value column, [B,T,HV,V]; p defaults to k.  With use_qk_l2norm_in_kernel q, k and p
    are normalised (fused_recurrent.py:90-93)."""
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if scale is None:
        scale = K ** -0.5
    if p is None:
        p = k
    qf, kf, pf, vf = q.to(dtype), k.to(dtype), p.to(dtype), v.to(dtype)
    if use_qk_l2norm_in_kernel:
        qf, kf, pf = (x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6) for x in (qf, kf, pf))
    qf, kf, pf = _expand_heads(qf, HV), _expand_heads(kf, HV), _expand_heads(pf, HV)
    bf = torch.ones(B, T, HV, dtype=dtype) if beta is None else beta.to(dtype)
    gf = g.to(dtype)
    if cu_seqlens is None:
        bounds = [(b, 0, T) for b in range(B)]
    else:
        cu = [int(x) for x in cu_seqlens]
        bounds = [(0, s, e) for s, e in zip(cu[:-1], cu[1:])]
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    ht = torch.zeros(len(bounds), HV, K, V, dtype=dtype)
    for n, (b, s, e) in enumerate(bounds):
        S = initial_state[n].to(dtype).clone() if initial_state is not None else torch.zeros(HV, K, V, dtype=dtype)
        for t in range(s, e):
            bt = bf[b, t] if bf.dim() == 4 else bf[b, t][:, None]          # a beta per value column (fused_recurrent.py:68-71, 97-100)
            vp = bt * (vf[b, t] - torch.einsum('hkv,hk->hv', S, pf[b, t]))
            S = S * gf[b, t].exp()[:, None, None] + kf[b, t][:, :, None] * vp[:, None, :]
            o[b, t] = torch.einsum('hkv,hk->hv', S, qf[b, t] * scale)
        ht[n] = S
    return o, (ht if output_final_state else None)


def chunk_comba_one_sequence(q, k, v, p, g, beta, scale, S0, chunk_size=64, dtype=torch.float32):
    """The comba operator in chunked form for one sequence and head (fla/ops/comba/naive.py:113-160; the kernels'
    stage order fla/ops/comba/chunk.py:22-90): with Gam the in-chunk cumsum of g and Gam0 = Gam - g,
        M_ij = (p_i . k_j) e^(Gam0_i - Gam_j) (i > j);  A = (I + diag(beta) M)^-1;  w = A (beta p e^Gam0);  u = A (beta v);
    then, as for the gated delta rule, v_new = u - w S;  o = scale (q e^Gam) S + scale tril(q k^T e^(Gam_i - Gam_j)) v_new;
    S <- e^Gam_last S + (k e^(Gam_last - Gam))^T v_new.
    q, k, p: [T,K]; v: [T,V]; g, beta: [T]; S0: [K,V].  Returns (o [T,V], S [K,V])."""
    T, K = k.shape
    q, k, v, p, g, beta = (x.to(dtype) for x in (q, k, v, p, g, beta))
    S = S0.to(dtype).clone()
    o = torch.zeros(T, v.shape[1], dtype=dtype)
    for t0 in range(0, T, chunk_size):
        sl = slice(t0, min(T, t0 + chunk_size))
        qc, kc, vc, pc, gc, bc = q[sl], k[sl], v[sl], p[sl], g[sl], beta[sl]
        n = qc.shape[0]
        gam = gc.cumsum(0)
        gam0 = gam - gc
        M = (pc @ kc.T) * (gam0[:, None] - gam[None, :]).tril(-1).exp().tril(-1)
        A = torch.linalg.solve_triangular(torch.eye(n, dtype=dtype) + bc[:, None] * M, torch.eye(n, dtype=dtype), upper=False)
        w = A @ (pc * (bc * gam0.exp())[:, None])
        u = A @ (vc * bc[:, None])
        v_new = u - w @ S
        P = scale * (qc @ kc.T) * (gam[:, None] - gam[None, :]).tril().exp().tril()
        o[sl] = scale * (qc * gam.exp()[:, None]) @ S + P @ v_new
        S = S * gam[-1].exp() + (kc * (gam[-1] - gam).exp()[:, None]).T @ v_new
    return o, S


def recurrent_gated_delta_rule_pooled(
    q, k, v, g, beta, scale, pool, ssm_state_indices, num_accepted_tokens=None, cu_seqlens=None,
    dtype=torch.float32, gk=None, **flags,
):
    """Token recurrence over states kept in a pool [num_slots,HV,K,V] (continuous batching and
    speculative decoding, fla/ops/kda/fused_recurrent.py:131-145,203-219).

    ssm_state_indices [N]: sequence n reads and finally rewrites slot [n].
    ssm_state_indices [N,Tmax]: sequence n starts from slot [n, num_accepted_tokens[n]-1] (entry 0
    without num_accepted_tokens) and the state after its token t is written to slot [n, t].
    Returns (o, pool after the call, states after every token [tokens,HV,K,V]).  Built on
    recurrent_gated_delta_rule, one token at a time, chained through its final state."""
    B, T = k.shape[:2]
    idx = torch.as_tensor(ssm_state_indices).long()
    bounds = [(b, 0, T) for b in range(B)] if cu_seqlens is None else \
        [(0, int(s), int(e)) for s, e in zip(cu_seqlens[:-1], cu_seqlens[1:])]
    pool_after = pool.to(dtype).clone()
    HV, V = v.shape[2], v.shape[3]
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    per_token = torch.zeros((B * T,) + tuple(pool.shape[1:]), dtype=dtype)
    for n, (b, s, e) in enumerate(bounds):
        if idx.dim() == 1:
            first = int(idx[n])
        else:
            first = int(idx[n, int(num_accepted_tokens[n]) - 1 if num_accepted_tokens is not None else 0])
        S = pool[first:first + 1].to(dtype)
        for t in range(s, e):
            sl = lambda x: None if x is None else x[b:b + 1, t:t + 1]
            o1, S = recurrent_gated_delta_rule(sl(q), sl(k), sl(v), sl(g), sl(beta), scale, S, True, dtype=dtype, gk=sl(gk), **flags)
            o[b, t] = o1[0, 0]
            per_token[b * T + t] = S[0]
            if idx.dim() == 2:
                pool_after[int(idx[n, t - s])] = S[0]
        if idx.dim() == 1 and e > s:
            pool_after[first] = S[0]
    return o, pool_after, per_token


# --------------------------------------------------------------------------- #
# chunked form, stage by stage
# --------------------------------------------------------------------------- #
def chunk_local_cumsum(g: torch.Tensor, chunk_size: int, cu_seqlens=None, scale: float | None = None,
                       reverse: bool = False) -> torch.Tensor:
    """Inclusive prefix sum of g [B,T,HV] restarted at every chunk of every
    sequence, optionally times ``scale`` (cumsum.py:33-68); fp32 result."""
    B, T, HV = g.shape
    out = torch.zeros(B, T, HV, dtype=torch.float32)
    bounds = [(b, 0, T) for b in range(B)] if cu_seqlens is None else \
        [(0, int(s), int(e)) for s, e in zip(cu_seqlens[:-1], cu_seqlens[1:])]
    for b, s, e in bounds:
        for c0 in range(s, e, chunk_size):
            c1 = min(c0 + chunk_size, e)
            seg = g[b, c0:c1].float()
            cs = seg.flip(0).cumsum(0).flip(0) if reverse else seg.cumsum(0)
            out[b, c0:c1] = cs * scale if scale is not None else cs
    return out


def chunk_stages_one_sequence(q, k, v, g, beta, scale, S0, chunk_size=64, dtype=torch.float32):
    """Chunk pipeline for ONE sequence and ONE v-head group already expanded:
    q,k [T,HV,K], v [T,HV,V], g,beta [T,HV], S0 [HV,K,V].  Returns a dict of every
    intermediate (per chunk lists) plus o [T,HV,V] and final S.

    Stage formulas (rows r of a chunk, G_r = cumsum(g)/ln2, gamma = 2^G):
      L[i,j] = beta_i (k_i.k_j) 2^(G_i-G_j), i>j;  A=(I+L)^-1     chunk_fwd.py:137-291
      u = A (beta*v);  w = A (beta*gamma*k)                        wy_fast.py:82-106
      v_new = u - w S;  S <- gamma_last S + k^T (v_new*2^(G_last-G))   chunk_delta_h.py:210-315
      o = scale[(q S) gamma + tril(q k^T 2^(G_i-G_j)) v_new]       chunk_o.py:107-153
    """
    T, HV, K = k.shape
    V = v.shape[-1]
    C = chunk_size
    q, k, v, g, beta = (x.to(dtype) for x in (q, k, v, g, beta))
    S = S0.to(dtype).clone()
    o = torch.zeros(T, HV, V, dtype=dtype)
    stages = dict(G=[], L=[], A=[], w=[], u=[], h=[], v_new=[])
    for c0 in range(0, T, C):
        c1 = min(c0 + C, T)
        r = c1 - c0
        kc, qc, vc = (x[c0:c1].transpose(0, 1) for x in (k, q, v))          # [HV,r,*]
        bc = beta[c0:c1].transpose(0, 1)                                     # [HV,r]
        G = g[c0:c1].transpose(0, 1).cumsum(-1) * RCP_LN2                    # [HV,r]
        diff = G[:, :, None] - G[:, None, :]
        strict = torch.ones(r, r, dtype=torch.bool).tril(-1)
        incl = torch.ones(r, r, dtype=torch.bool).tril(0)
        # mask BEFORE exponentiating so the upper triangle cannot overflow
        dec_strict = torch.where(strict, torch.exp2(torch.where(strict, diff, torch.zeros_like(diff))), torch.zeros_like(diff))
        dec_incl = torch.where(incl, torch.exp2(torch.where(incl, diff, torch.zeros_like(diff))), torch.zeros_like(diff))
        L = bc[:, :, None] * (kc @ kc.transpose(-1, -2)) * dec_strict
        eye = torch.eye(r, dtype=dtype).expand(HV, r, r)
        A = torch.linalg.solve_triangular(eye + L, eye.clone(), upper=False, unitriangular=True)
        gamma = torch.exp2(G)
        u = A @ (vc * bc[:, :, None])
        w = A @ (kc * (bc * gamma)[:, :, None])
        v_new = u - w @ S
        o_c = (qc @ S) * gamma[:, :, None] + ((qc @ kc.transpose(-1, -2)) * dec_incl) @ v_new
        o[c0:c1] = (o_c * scale).transpose(0, 1)
        stages['G'].append(G); stages['L'].append(L); stages['A'].append(A)
        stages['w'].append(w); stages['u'].append(u); stages['h'].append(S.clone()); stages['v_new'].append(v_new)
        g_last = G[:, -1]
        S = S * torch.exp2(g_last)[:, None, None] + \
            (kc * torch.exp2(g_last[:, None] - G)[:, :, None]).transpose(-1, -2) @ v_new
    stages['o'] = o
    stages['S'] = S
    return stages


def chunk_gated_delta_rule(
    q, k, v, g, beta, scale=None, initial_state=None, output_final_state=False,
    cu_seqlens=None, chunk_size=64,
    use_qk_l2norm_in_kernel=False, use_gate_in_kernel=False, A_log=None, dt_bias=None,
    use_beta_sigmoid_in_kernel=False, allow_neg_eigval=False, state_v_first=False,
    dtype=torch.float32, return_stages=False,
):
    """Chunked gated delta rule with the argument order of
    fla/ops/gated_delta_rule/chunk.py:397-415 (q, k, v, g, beta).  Returns
    (o [B,T,HV,V], final_state [N,HV,K,V] or None) in ``dtype``."""
    B, T, H, K = k.shape
    HV, V = v.shape[2], v.shape[3]
    if scale is None:
        scale = K ** -0.5
    qf, kf, vf = q.to(dtype), k.to(dtype), v.to(dtype)
    if use_qk_l2norm_in_kernel:
        # chunk.py:279-282 normalises through l2norm_fwd, whose output keeps the input dtype
        qf = l2norm(q).to(q.dtype).to(dtype)
        kf = l2norm(k).to(k.dtype).to(dtype)
    qf, kf = _expand_heads(qf, HV), _expand_heads(kf, HV)
    bf = beta.to(dtype)
    if use_beta_sigmoid_in_kernel:
        bf = torch.sigmoid(bf) * (2.0 if allow_neg_eigval else 1.0)
    gf = gdn_gate(g, A_log, dt_bias).to(dtype) if use_gate_in_kernel else g.to(dtype)

    if cu_seqlens is None:
        bounds = [(b, 0, T) for b in range(B)]
    else:
        cu = [int(x) for x in cu_seqlens]
        bounds = [(0, s, e) for s, e in zip(cu[:-1], cu[1:])]
    N = len(bounds)
    o = torch.zeros(B, T, HV, V, dtype=dtype)
    ht = torch.zeros(N, HV, K, V, dtype=dtype)
    all_stages = []
    for n, (b, s, e) in enumerate(bounds):
        S0 = torch.zeros(HV, K, V, dtype=dtype)
        if initial_state is not None:
            S0 = initial_state[n].to(dtype)
            if state_v_first:
                S0 = S0.transpose(-1, -2)
        st = chunk_stages_one_sequence(qf[b, s:e], kf[b, s:e], vf[b, s:e], gf[b, s:e], bf[b, s:e],
                                       scale, S0, chunk_size, dtype)
        o[b, s:e] = st['o']
        ht[n] = st['S']
        all_stages.append(st)
    fs = None
    if output_final_state:
        fs = ht.transpose(-1, -2).contiguous() if state_v_first else ht
    if return_stages:
        return o, fs, all_stages
    return o, fs


# --------------------------------------------------------------------------- #
# one decode step in closed form (used to pin the recurrence and as the CPU
# baseline of the decode bench): S' = e^g S + k [beta (v - e^g S^T k)]^T, o = scale S'^T q
# --------------------------------------------------------------------------- #
def decode_step(q, k, v, g, beta, S, scale=None):
    """q,k [N,H,K]; v [N,HV,V]; g,beta [N,HV]; S [N,HV,K,V] fp32.  Vectorised over
    N and HV.  Returns (o [N,HV,V], S' [N,HV,K,V])."""
    N, H, K = k.shape
    HV = v.shape[1]
    if scale is None:
        scale = K ** -0.5
    G = HV // H
    qf = q.float().repeat_interleave(G, dim=1)
    kf = k.float().repeat_interleave(G, dim=1)
    S = S.float() * g.float().exp()[:, :, None, None]
    vp = beta.float()[:, :, None] * (v.float() - torch.einsum('nhkv,nhk->nhv', S, kf))
    S = S + kf[:, :, :, None] * vp[:, :, None, :]
    o = torch.einsum('nhkv,nhk->nhv', S, qf * scale)
    return o, S


def make_inputs(B, T, H, HV, K, V, seed=42, gate_div=1.0, h0_std=None, N=None, dtype=torch.float32):
    """Synthetic inputs in the order q,k,v,g,beta,h0 from one CPU generator:
    q,k = normalize(randn), v = randn, g = logsigmoid(randn)/gate_div,
    beta = sigmoid(randn), h0 = h0_std*randn or None.  q,k,v are cast to ``dtype``
    (g, beta, h0 stay fp32)."""
    gen = torch.Generator().manual_seed(seed)
    q = F.normalize(torch.randn(B, T, H, K, generator=gen), p=2, dim=-1)
    k = F.normalize(torch.randn(B, T, H, K, generator=gen), p=2, dim=-1)
    v = torch.randn(B, T, HV, V, generator=gen)
    g = F.logsigmoid(torch.randn(B, T, HV, generator=gen)) / gate_div
    beta = torch.sigmoid(torch.randn(B, T, HV, generator=gen))
    h0 = None
    if h0_std is not None:
        h0 = h0_std * torch.randn(N if N is not None else B, HV, K, V, generator=gen)
    return q.to(dtype), k.to(dtype), v.to(dtype), g, beta, h0


def make_varlen_lengths(total: int, n_seq: int, lo: int, hi: int, seed: int = 42) -> list[int]:
    """Lengths ~ U[lo,hi] rescaled (floor) to sum to ``total``; the remainder is
    handed out one token at a time to the first sequences."""
    gen = torch.Generator().manual_seed(seed)
    L = torch.randint(lo, hi + 1, (n_seq,), generator=gen).double()
    L = torch.floor(L * total / L.sum()).long()
    rem = total - int(L.sum())
    for i in range(rem):
        L[i % n_seq] += 1
    assert int(L.sum()) == total and int(L.min()) >= 1
    return [int(x) for x in L]


# --------------------------------------------------------------------------- #
# backward
# --------------------------------------------------------------------------- #
def gated_delta_rule_grads(
    q, k, v, g, beta, do, dht=None, scale=None, initial_state=None, cu_seqlens=None,
    use_qk_l2norm_in_kernel=False, use_gate_in_kernel=False, A_log=None, dt_bias=None,
    use_beta_sigmoid_in_kernel=False, allow_neg_eigval=False, state_v_first=False,
    dtype=torch.float64,
):
    """Gradients of  sum(o * do) + sum(ht * dht)  with respect to q, k, v, g, beta, the initial state and
    (with the gate activation) A_log and dt_bias, by reverse-mode differentiation of the token recurrence
    above: what the reference's own tests take as the truth for its backward pass
    (tests/ops/test_gdn.py:160-176, autograd through the naive implementation).  Returns a dict with
    the keys dq, dk, dv, dg, dbeta, dh0, dA_log, ddt_bias (None where there is no such input)."""
    leaves = {}

    def leaf(name, x):
        if x is None:
            return None
        leaves[name] = x.detach().to(dtype).clone().requires_grad_(True)
        return leaves[name]

    q_, k_, v_, g_, b_ = leaf('dq', q), leaf('dk', k), leaf('dv', v), leaf('dg', g), leaf('dbeta', beta)
    h0_ = leaf('dh0', initial_state)
    A_ = leaf('dA_log', A_log) if use_gate_in_kernel else None
    dt_ = leaf('ddt_bias', dt_bias) if use_gate_in_kernel else None
    o, ht = recurrent_gated_delta_rule(
        q_, k_, v_, g_, b_, scale=scale, initial_state=h0_, output_final_state=dht is not None, cu_seqlens=cu_seqlens,
        use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, use_gate_in_kernel=use_gate_in_kernel, A_log=A_, dt_bias=dt_,
        use_beta_sigmoid_in_kernel=use_beta_sigmoid_in_kernel, allow_neg_eigval=allow_neg_eigval,
        state_v_first=state_v_first, dtype=dtype)
    loss = (o * do.to(dtype)).sum()
    if dht is not None:
        loss = loss + (ht * dht.to(dtype)).sum()
    names = list(leaves)
    grads = torch.autograd.grad(loss, [leaves[n] for n in names], allow_unused=True)
    out = dict.fromkeys(('dq', 'dk', 'dv', 'dg', 'dbeta', 'dh0', 'dA_log', 'ddt_bias'))
    out.update(dict(zip(names, grads)))
    return out


def kda_grads(q, k, v, g, beta, do, dht=None, scale=None, initial_state=None, cu_seqlens=None,
              use_qk_l2norm_in_kernel=False, use_gate_in_kernel=False, A_log=None, dt_bias=None, lower_bound=None,
              use_beta_sigmoid_in_kernel=False, allow_neg_eigval=False, state_v_first=False, dtype=torch.float64):
    """Gradients of  sum(o * do) + sum(ht * dht)  of the KDA operator with respect to q, k, v, g, beta, the initial state
    and (with the gate activation) A_log and dt_bias, by reverse-mode differentiation of ``recurrent_kda``: what the
    reference's tests take as the truth for chunk_kda's backward pass (tests/ops/test_kda.py, autograd through
    fla/ops/kda/naive.py).  Returns a dict with the keys dq, dk, dv, dg, dbeta, dh0, dA_log, ddt_bias."""
    leaves = {}
    gate = dict(dA_log=A_log, ddt_bias=dt_bias) if use_gate_in_kernel else {}
    for name, x in dict(dq=q, dk=k, dv=v, dg=g, dbeta=beta, dh0=initial_state, **gate).items():
        leaves[name] = None if x is None else x.detach().to(dtype).clone().requires_grad_(True)
    o, ht = recurrent_kda(leaves['dq'], leaves['dk'], leaves['dv'], leaves['dg'], leaves['dbeta'], scale=scale,
                          initial_state=leaves['dh0'], output_final_state=dht is not None, cu_seqlens=cu_seqlens,
                          use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, use_gate_in_kernel=use_gate_in_kernel,
                          A_log=leaves.get('dA_log'), dt_bias=leaves.get('ddt_bias'), lower_bound=lower_bound,
                          use_beta_sigmoid_in_kernel=use_beta_sigmoid_in_kernel, allow_neg_eigval=allow_neg_eigval,
                          state_v_first=state_v_first, dtype=dtype)
    loss = (o * do.to(dtype)).sum()
    if dht is not None:
        loss = loss + (ht * dht.to(dtype)).sum()
    names = [n for n, x in leaves.items() if x is not None]
    grads = torch.autograd.grad(loss, [leaves[n] for n in names], allow_unused=True)
    out = dict.fromkeys(('dq', 'dk', 'dv', 'dg', 'dbeta', 'dh0', 'dA_log', 'ddt_bias'))
    out.update(dict(zip(names, grads)))
    return out


def comba_grads(q, k, v, p, g, beta, do, dht=None, scale=None, initial_state=None, cu_seqlens=None,
                use_qk_l2norm_in_kernel=False, dtype=torch.float64):
    """Gradients of  sum(o * do) + sum(ht * dht)  of the comba operator with respect to q, k, v, p, g, beta and the
    initial state, by reverse-mode differentiation of ``recurrent_comba``: what the reference's tests take as the
    truth for chunk_comba's backward pass (tests/ops/test_comba.py:92-150, autograd through fla/ops/comba/naive.py,
    the same map).  Returns a dict with the keys dq, dk, dv, dp, dg, dbeta, dh0 (None where there is no such input)."""
    leaves = {}
    for name, x in dict(dq=q, dk=k, dv=v, dp=p, dg=g, dbeta=beta, dh0=initial_state).items():
        leaves[name] = None if x is None else x.detach().to(dtype).clone().requires_grad_(True)
    o, ht = recurrent_comba(leaves['dq'], leaves['dk'], leaves['dv'], leaves['dp'], leaves['dg'], leaves['dbeta'], scale=scale,
                            initial_state=leaves['dh0'], output_final_state=dht is not None, cu_seqlens=cu_seqlens,
                            use_qk_l2norm_in_kernel=use_qk_l2norm_in_kernel, dtype=dtype)
    loss = (o * do.to(dtype)).sum()
    if dht is not None:
        loss = loss + (ht * dht.to(dtype)).sum()
    names = [n for n, x in leaves.items() if x is not None]
    grads = torch.autograd.grad(loss, [leaves[n] for n in names], allow_unused=True)
    out = dict.fromkeys(leaves)
    out.update(dict(zip(names, grads)))
    return out


def chunk_backward_one_sequence(q, k, v, g, beta, scale, S0, do, dSt=None, chunk_size=64, dtype=torch.float64):
    """The reference's chunked backward pass, stage by stage, for ONE sequence with the q/k heads already
    expanded: q, k [T,HV,K]; v, do [T,HV,V]; g, beta [T,HV]; S0 [HV,K,V]; dSt [HV,K,V] or None.
    Natural-log gates (gam_r = cumsum(g) inside the chunk).  Returns the gradients and every intermediate.

    Stages (fla/ops/gated_delta_rule/chunk.py:125-257):
      recompute  A, w = A (beta e^gam k), u = A (beta v); states S_c and v_new = u - w S_c    wy_fast.py:72-106, chunk_delta_h.py:174-348
      reverse scan over chunks (chunk_delta_h.py:369-560, chunk_o.py:465-560):
        dv_new = P^T do + (k e^(gam_last - gam)) dS_next,      P = scale tril(q k^T e^(gam_i - gam_j))
        dS     = e^gam_last dS_next + scale (q e^gam)^T do - w^T dv_new
      per chunk (chunk_o.py:172-357):
        dq = scale e^gam (do S^T) + (dP o D) k,  dk = (dP o D)^T q + e^(gam_last - gam) (v_new dS_next^T),
        dw = -dv_new S^T,   dP = scale tril(do v_new^T),  D_ij = e^(gam_i - gam_j)
        dgam from every factor e^gam above; dgam_last also from e^gam_last <S, dS_next>
      WY factors backwards (wy_fast.py:123-296):  X = A diag(beta)
        dX = tril(dw (e^gam k)^T + du v^T),  d(e^gam k) = X^T dw,  dv = X^T du,
        dL = -stril(A^T (dX diag(beta)) A^T),  L = diag(beta) stril(k k^T o D)
      dg = reverse cumulative sum of dgam inside the chunk (cumsum.py, reverse=True)."""
    T, HV, K = k.shape
    V = v.shape[-1]
    C = chunk_size
    q, k, v, g, beta, do = (x.to(dtype) for x in (q, k, v, g, beta, do))
    NT = (T + C - 1) // C
    fwd = []
    S = S0.to(dtype).clone()
    for ic in range(NT):
        c0, c1 = ic * C, min(ic * C + C, T)
        r = c1 - c0
        kc, qc, vc, doc = (x[c0:c1].transpose(0, 1) for x in (k, q, v, do))      # [HV,r,*]
        bc = beta[c0:c1].transpose(0, 1)
        gam = g[c0:c1].transpose(0, 1).cumsum(-1)                               # [HV,r]
        diff = gam[:, :, None] - gam[:, None, :]
        incl = torch.ones(r, r, dtype=torch.bool).tril(0)
        strict = torch.ones(r, r, dtype=torch.bool).tril(-1)
        D = torch.where(incl, torch.exp(torch.where(incl, diff, torch.zeros_like(diff))), torch.zeros_like(diff))
        KK = kc @ kc.transpose(-1, -2)
        M = torch.where(strict, KK * D, torch.zeros_like(D))
        eye = torch.eye(r, dtype=dtype).expand(HV, r, r)
        A = torch.linalg.solve_triangular(eye + bc[:, :, None] * M, eye.clone(), upper=False, unitriangular=True)
        eg = gam.exp()
        w = A @ (kc * (bc * eg)[:, :, None])
        u = A @ (vc * bc[:, :, None])
        vn = u - w @ S
        P = scale * (qc @ kc.transpose(-1, -2)) * D
        glast = gam[:, -1]
        kb = kc * torch.exp(glast[:, None] - gam)[:, :, None]
        fwd.append(dict(c0=c0, c1=c1, kc=kc, qc=qc, vc=vc, doc=doc, bc=bc, gam=gam, D=D, M=M, A=A, w=w, u=u, vn=vn, P=P,
                        S=S.clone(), glast=glast, kb=kb, eg=eg, incl=incl, strict=strict))
        S = S * glast.exp()[:, None, None] + kb.transpose(-1, -2) @ vn
    dS = torch.zeros(HV, K, V, dtype=dtype) if dSt is None else dSt.to(dtype).clone()
    dq, dk, dv = torch.zeros_like(q), torch.zeros_like(k), torch.zeros_like(v)
    dg, dbeta = torch.zeros_like(g), torch.zeros_like(beta)
    stages = [None] * NT
    for ic in reversed(range(NT)):
        f = fwd[ic]
        kc, qc, vc, doc, bc, gam, D, M, A, w, vn, P, Sc, glast, kb, eg = (f[n] for n in (
            'kc', 'qc', 'vc', 'doc', 'bc', 'gam', 'D', 'M', 'A', 'w', 'vn', 'P', 'S', 'glast', 'kb', 'eg'))
        dSn = dS
        dvn = P.transpose(-1, -2) @ doc + kb @ dSn
        dS = dSn * glast.exp()[:, None, None] + scale * (qc * eg[:, :, None]).transpose(-1, -2) @ doc - w.transpose(-1, -2) @ dvn
        # per chunk
        dPm = torch.where(f['incl'], scale * (doc @ vn.transpose(-1, -2)) * D, torch.zeros_like(D))
        dq_c = scale * eg[:, :, None] * (doc @ Sc.transpose(-1, -2)) + dPm @ kc
        dk_P = dPm.transpose(-1, -2) @ qc
        dk_S = torch.exp(glast[:, None] - gam)[:, :, None] * (vn @ dSn.transpose(-1, -2))
        dw = -dvn @ Sc.transpose(-1, -2)
        dgam = (qc * dq_c).sum(-1) - (kc * (dk_P + dk_S)).sum(-1)
        dgam[:, -1] += glast.exp() * (Sc * dSn).sum((-1, -2)) + (kc * dk_S).sum((-1, -2))
        # WY factors
        X = A * bc[:, None, :]
        kd = kc * eg[:, :, None]
        dX = torch.where(f['incl'], dw @ kd.transpose(-1, -2) + dvn @ vc.transpose(-1, -2), torch.zeros_like(D))
        dkd = X.transpose(-1, -2) @ dw
        dv_c = X.transpose(-1, -2) @ dvn
        dk_c = dq_c.new_zeros(kc.shape) + dk_P + dk_S + dkd * eg[:, :, None]
        dgam = dgam + (kd * dkd).sum(-1)
        db = (dX * A).sum(-2)
        dA = dX * bc[:, None, :]
        dL = torch.where(f['strict'], -(A.transpose(-1, -2) @ dA @ A.transpose(-1, -2)), torch.zeros_like(D))
        db = db + (dL * M).sum(-1)
        E = dL * bc[:, :, None] * D
        dk_c = dk_c + E @ kc + E.transpose(-1, -2) @ kc
        F_ = E * (kc @ kc.transpose(-1, -2))
        dgam = dgam + F_.sum(-1) - F_.sum(-2)
        c0, c1 = f['c0'], f['c1']
        dq[c0:c1] = dq_c.transpose(0, 1)
        dk[c0:c1] = dk_c.transpose(0, 1)
        dv[c0:c1] = dv_c.transpose(0, 1)
        dbeta[c0:c1] = db.transpose(0, 1)
        dg[c0:c1] = dgam.flip(-1).cumsum(-1).flip(-1).transpose(0, 1)
        stages[ic] = dict(A=A, w=w, u=f['u'], S=Sc, vn=vn, P=P, dvn=dvn, dSn=dSn, dw=dw, dgam=dgam)
    return dict(dq=dq, dk=dk, dv=dv, dg=dg, dbeta=dbeta, dh0=dS, stages=stages)
