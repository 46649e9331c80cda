"""CPU oracle for the two steps either side of the gated delta rule in the layer: the causal short
convolution and the gated normalisation.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this module: it is the checker used
by ``tests/`` and the ``cpu_baseline`` leg of ``bench.py``.  It restates, in plain torch CPU ops, the
algorithm of the reference's files (paths relative to the reference checkout):

* ``fla/modules/conv/triton/kernels.py:37-139``   causal_conv1d_fwd_kernel: taps, initial state, bias,
  activation, residual - in that order
* ``fla/modules/conv/triton/kernels.py:520-582``  causal_conv1d_states_fwd_kernel: the state after a prefill
* ``fla/modules/conv/triton/kernels.py:356-421``  causal_conv1d_update_kernel: one-token update of the cache
* ``fla/modules/fused_norm_gate.py:36-108``       layer_norm_gated_fwd_kernel: residual, statistics, affine, gate

Parity pins (all in ``tests/test_oracle_modules.py``): ``torch.nn.functional.conv1d`` with causal padding
(the routine the reference's own tests compare with, tests/modules/test_conv.py:30-72), a scalar pure-python
loop on tiny shapes, prefill split in two with the state handed over == one prefill, T one-token updates ==
one prefill, packed == per-sequence loop; ``F.layer_norm`` / ``F.rms_norm`` times the gate for the
normalisation.  No function here is "parity unpinned".

Everything is computed in ``dtype`` (float32 by default); inputs are upcast first and results are NOT rounded
back, so a kernel's output is compared with the exact value of the formula on its rounded inputs.
"""
from __future__ import annotations

import torch


def _silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def causal_conv1d(x, weight, bias=None, residual=None, initial_state=None, output_final_state=False,
                  activation=None, cu_seqlens=None, dtype=torch.float32):
    """x [B,T,D], weight [D,W], bias [D], residual [B,T,D], initial_state [N,D,W] -> (y [B,T,D], final [N,D,W] | None).

    y[t] = act(sum_j weight[:, j] * x[t - (W-1) + j] + bias) + residual[t]; positions p < 0 of a sequence read
    initial_state[n, :, W + p] (entry 0 is never used).  final[n, :, w] = input at position len - W + w.
    """
    assert activation in (None, 'silu', 'swish')
    B, T, D = x.shape
    W = weight.shape[1]
    xs = x.to(dtype)
    wt = weight.to(dtype)
    if cu_seqlens is None:
        bounds = [(b, 0, T) for b in range(B)]
    else:
        assert B == 1
        cu = [int(c) for c in cu_seqlens]
        bounds = [(0, cu[i], cu[i + 1]) for i in range(len(cu) - 1)]
    y = torch.zeros(B, T, D, dtype=dtype)
    final = torch.zeros(len(bounds), D, W, dtype=dtype) if output_final_state else None
    for n, (b, bos, eos) in enumerate(bounds):
        L = eos - bos
        # the sequence with its W positions of history in front: ext[W + p] = input at position p
        hist = initial_state[n].to(dtype).T if initial_state is not None else torch.zeros(W, D, dtype=dtype)
        ext = torch.cat([hist, xs[b, bos:eos]], dim=0)
        acc = torch.zeros(L, D, dtype=dtype)
        for j in range(W):
            # tap j multiplies position t - (W-1) + j, i.e. ext row t + 1 + j
            acc += ext[1 + j:1 + j + L] * wt[:, j]
        if bias is not None:
            acc += bias.to(dtype)
        if activation is not None:
            acc = _silu(acc)
        if residual is not None:
            acc += residual[b, bos:eos].to(dtype)
        y[b, bos:eos] = acc
        if final is not None:
            final[n] = ext[L:L + W].T
    return y, final


def causal_conv1d_update(x, cache, weight, bias=None, residual=None, activation=None, dtype=torch.float32):
    """One token per sequence: x [N,D], cache [N,D,W] -> (y [N,D], new cache [N,D,W]) - the cache moves one place
    to the left and takes x as its last entry, then is contracted with the weight."""
    assert activation in (None, 'silu', 'swish')
    new_cache = torch.cat([cache.to(dtype)[:, :, 1:], x.to(dtype)[:, :, None]], dim=-1)
    y = (new_cache * weight.to(dtype)).sum(-1)
    if bias is not None:
        y = y + bias.to(dtype)
    if activation is not None:
        y = _silu(y)
    if residual is not None:
        y = y + residual.to(dtype)
    return y, new_cache


def norm_gated(x, g, weight=None, bias=None, residual=None, eps=1e-5, activation='swish', is_rms_norm=False,
               dtype=torch.float32):
    """Rows of x [T,D]: r = x + residual; y = (r - mean) * rstd * weight + bias, gated by g * sigmoid(g) (swish)
    or sigmoid(g).  Returns (y, r, mean, rstd); mean is zero for RMS norm."""
    assert activation in ('swish', 'silu', 'sigmoid')
    r = x.to(dtype)
    if residual is not None:
        r = r + residual.to(dtype)
    if is_rms_norm:
        mean = torch.zeros(r.shape[0], dtype=dtype)
        var = (r * r).mean(-1)
    else:
        mean = r.mean(-1)
        var = ((r - mean[:, None]) ** 2).mean(-1)
    rstd = 1.0 / torch.sqrt(var + eps)
    y = (r - mean[:, None]) * rstd[:, None]
    if weight is not None:
        y = y * weight.to(dtype)
    if bias is not None:
        y = y + bias.to(dtype)
    gg = g.to(dtype)
    y = y * gg * torch.sigmoid(gg) if activation in ('swish', 'silu') else y * torch.sigmoid(gg)
    return y, r, mean, rstd


def conv_grads(x, weight, bias, residual, initial_state, dy, dht=None, activation=None, cu_seqlens=None, dtype=torch.float64):
    """Gradients of ``causal_conv1d`` for the output gradients (dy, dht): reverse-mode differentiation of the oracle's own
    forward in ``dtype`` (fla/modules/conv/triton/ops.py:147-249 computes the same quantities).  Returns a dict with
    dx, dw, db, dr, dh0 (None where the input is absent)."""
    leaves = {}
    for name, t in (('x', x), ('w', weight), ('b', bias), ('r', residual), ('h0', initial_state)):
        leaves[name] = None if t is None else t.detach().to(dtype).clone().requires_grad_(True)
    y, final = causal_conv1d(leaves['x'], leaves['w'], leaves['b'], leaves['r'], leaves['h0'], dht is not None,
                             activation, cu_seqlens, dtype)
    loss = (y * dy.to(dtype)).sum()
    if dht is not None:
        loss = loss + (final * dht.to(dtype)).sum()
    loss.backward()
    return {('d' + k): (None if v is None else v.grad) for k, v in leaves.items()}


def norm_gated_grads(x, g, weight, bias, residual, dy, dres_out=None, eps=1e-5, activation='swish', is_rms_norm=False,
                     dtype=torch.float64):
    """Gradients of ``norm_gated`` for the gradient dy of y and (prenorm) dres_out of the residual stream r:
    reverse-mode differentiation of the oracle's own forward (fla/modules/fused_norm_gate.py:541-650 computes the same).
    Returns a dict with dx, dg, dw, db, dr."""
    leaves = {}
    for name, t in (('x', x), ('g', g), ('w', weight), ('b', bias), ('r', residual)):
        leaves[name] = None if t is None else t.detach().to(dtype).clone().requires_grad_(True)
    y, r, _, _ = norm_gated(leaves['x'], leaves['g'], leaves['w'], leaves['b'], leaves['r'], eps, activation, is_rms_norm, dtype)
    loss = (y * dy.to(dtype)).sum()
    if dres_out is not None:
        loss = loss + (r * dres_out.to(dtype)).sum()
    loss.backward()
    return {('d' + k): (None if v is None else v.grad) for k, v in leaves.items()}
