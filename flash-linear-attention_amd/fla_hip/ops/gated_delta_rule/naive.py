"""Plain-torch forms of the gated delta rule with the public names and argument orders of
fla/ops/gated_delta_rule/naive.py:13-64 (token recurrence; note ``(q, k, v, beta, g)``) and
:67-161 (chunked; ``(q, k, v, g, beta)``).  They run on any device torch runs on, need
``H == HV``, compute in fp32 and exist for checking and for CPU timing; the HIP operators
never call them."""
from __future__ import annotations

import torch
import torch.nn.functional as F


def naive_recurrent_gated_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    beta: torch.Tensor,
    g: torch.Tensor,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
):
    """q, k ``[B,T,H,K]``; v ``[B,T,H,V]``; beta, g ``[B,T,H]``; state ``[B,H,K,V]``."""
    B, T, H, K = k.shape
    V = v.shape[-1]
    if scale is None:
        scale = K ** -0.5
    qf, kf, vf, bf, gf = (x.float() for x in (q, k, v, beta, g))
    S = torch.zeros(B, H, K, V, dtype=torch.float32, device=v.device) if initial_state is None \
        else initial_state.float().clone()
    o = torch.empty(B, T, H, V, dtype=torch.float32, device=v.device)
    decay = gf.exp()
    for t in range(T):
        S = S * decay[:, t, :, None, None]
        delta = bf[:, t, :, None] * (vf[:, t] - torch.einsum('bhkv,bhk->bhv', S, kf[:, t]))
        S = S + kf[:, t, :, :, None] * delta[:, :, None, :]
        o[:, t] = torch.einsum('bhkv,bhk->bhv', S, qf[:, t]) * scale
    return o, (S if output_final_state else None)


def naive_chunk_gated_delta_rule(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    g: torch.Tensor,
    beta: torch.Tensor,
    chunk_size: int = 64,
    scale: float = None,
    initial_state: torch.Tensor = None,
    output_final_state: bool = False,
):
    """Chunked evaluation (WY form).  T is zero-padded to a multiple of ``chunk_size``."""
    B, T, H, K = k.shape
    V = v.shape[-1]
    C = chunk_size
    if scale is None:
        scale = K ** -0.5
    pad = (-T) % C
    # head-major fp32 working copies [B,H,T,*]
    qf, kf, vf = (F.pad(x.float().transpose(1, 2), (0, 0, 0, pad)) for x in (q, k, v))
    bf, gf = (F.pad(x.float().transpose(1, 2), (0, pad)) for x in (beta, g))
    NT = (T + pad) // C
    qf, kf, vf = (x.reshape(B, H, NT, C, -1) for x in (qf, kf, vf))
    bf, G = bf.reshape(B, H, NT, C), gf.reshape(B, H, NT, C).cumsum(-1)
    dev = v.device
    lower = torch.ones(C, C, dtype=torch.bool, device=dev).tril(-1)
    lower_eq = torch.ones(C, C, dtype=torch.bool, device=dev).tril(0)
    diff = (G[..., :, None] - G[..., None, :]).masked_fill(~lower_eq, 0.0)
    decay = diff.exp().masked_fill(~lower_eq, 0.0)                           # e^{G_i-G_j}, i >= j
    eye = torch.eye(C, device=dev)
    L = (bf[..., None] * (kf @ kf.transpose(-1, -2)) * decay).masked_fill(~lower, 0.0)
    A = torch.linalg.solve_triangular(eye + L, eye.expand_as(L).contiguous(), upper=False, unitriangular=True)
    u = A @ (vf * bf[..., None])
    w = A @ (kf * (bf * G.exp())[..., None])
    S = torch.zeros(B, H, K, V, dtype=torch.float32, device=dev) if initial_state is None \
        else initial_state.float().clone()
    o = torch.empty(B, H, NT, C, V, dtype=torch.float32, device=dev)
    for c in range(NT):
        v_new = u[:, :, c] - w[:, :, c] @ S
        attn = (qf[:, :, c] @ kf[:, :, c].transpose(-1, -2)) * decay[:, :, c]
        o[:, :, c] = scale * ((qf[:, :, c] * G[:, :, c, :, None].exp()) @ S + attn @ v_new)
        tail = (G[:, :, c, -1:] - G[:, :, c]).exp()
        S = S * G[:, :, c, -1, None, None].exp() + (kf[:, :, c] * tail[..., None]).transpose(-1, -2) @ v_new
    o = o.reshape(B, H, NT * C, V)[:, :, :T].transpose(1, 2)
    return o, (S if output_final_state else None)
