"""Plain-torch forms of the comba operator with the public names and argument orders of fla/ops/comba/naive.py:13-67
(token loop; note ``(q, k, v, p, beta, g)``) and :70-171 (chunked; ``(q, k, v, p, g, beta)``).  They run on any device torch
runs on, need ``H == HV``, compute in fp32 and exist for checking; the HIP operators never call them.

The two are NOT the same map, here as in the reference: the chunked form - the one the reference's tests take as the truth
and the one ``chunk_comba`` / ``fused_recurrent_comba`` compute - predicts with p from the state BEFORE the token's decay;
the token loop decays first."""
from __future__ import annotations

import torch


def naive_recurrent_comba(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    p: torch.Tensor,
    beta: torch.Tensor,
    g: torch.Tensor,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
):
    """q, k, p ``[B,T,H,K]``; v ``[B,T,H,V]``; beta, g ``[B,T,H]``; state ``[B,H,K,V]``.  Per token:
    S <- e^g S;  v' = beta (v - S^T p);  S <- S + k v'^T;  o = scale S^T q."""
    B, T, H, K = k.shape
    V = v.shape[-1]
    if scale is None:
        scale = K ** -0.5
    qf, kf, vf, pf, bf, gf = (x.float() for x in (q, k, v, p, beta, g))
    S = torch.zeros(B, H, K, V, dtype=torch.float32, device=v.device) if initial_state is None else initial_state.float().clone()
    o = torch.empty(B, T, H, V, dtype=torch.float32, device=v.device)
    for t in range(T):
        S = S * gf[:, t].exp()[..., None, None]
        delta = bf[:, t, :, None] * (vf[:, t] - torch.einsum('bhkv,bhk->bhv', S, pf[:, t]))
        S = S + kf[:, t, :, :, None] * delta[:, :, None, :]
        o[:, t] = torch.einsum('bhkv,bhk->bhv', S, qf[:, t]) * scale
    return o, (S if output_final_state else None)


def naive_chunk_comba(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    p: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    chunk_size: int = 64,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
):
    """Chunked form: with Gam the in-chunk running sum of g and Gam0 = Gam - g,
    A = (I + diag(beta) stril((p k^T) e^(Gam0_i - Gam_j)))^-1,  w = A (beta p e^Gam0),  u = A (beta v);  per chunk
    v_new = u - w S;  o = scale (q e^Gam) S + scale tril((q k^T) e^(Gam_i - Gam_j)) v_new;  S <- e^Gam_last S + (k e^(Gam_last - Gam))^T v_new."""
    B, T, H, K = k.shape
    V = v.shape[-1]
    if scale is None:
        scale = K ** -0.5
    qf, kf, vf, pf, gf, bf = (x.float().transpose(1, 2) for x in (q, k, v, p, g, beta))     # [B,H,T,...]
    S = torch.zeros(B, H, K, V, dtype=torch.float32, device=v.device) if initial_state is None else initial_state.float().clone()
    o = torch.empty(B, H, T, V, dtype=torch.float32, device=v.device)
    for t0 in range(0, T, chunk_size):
        sl = slice(t0, min(T, t0 + chunk_size))
        qc, kc, vc, pc, gc, bc = qf[:, :, sl], kf[:, :, sl], vf[:, :, sl], pf[:, :, sl], gf[:, :, sl], bf[:, :, sl]
        n = qc.shape[2]
        gam = gc.cumsum(-1)
        gam0 = gam - gc
        eye = torch.eye(n, dtype=torch.float32, device=v.device)
        M = (pc @ kc.transpose(-1, -2)) * (gam0[..., :, None] - gam[..., None, :]).tril(-1).exp().tril(-1)
        A = torch.linalg.solve_triangular(eye + bc[..., None] * M, eye.expand(B, H, n, n), upper=False)
        w = A @ (pc * (bc * gam0.exp())[..., None])
        u = A @ (vc * bc[..., None])
        v_new = u - w @ S
        P = (qc @ kc.transpose(-1, -2)) * (gam[..., :, None] - gam[..., None, :]).tril().exp().tril()
        o[:, :, sl] = scale * ((qc * gam.exp()[..., None]) @ S + P @ v_new)
        S = S * gam[..., -1, None, None].exp() + (kc * (gam[..., -1:] - gam).exp()[..., None]).transpose(-1, -2) @ v_new
    return o.transpose(1, 2), (S if output_final_state else None)
