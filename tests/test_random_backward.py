"""Seeded random combinations for the three chunked operators' backward passes (gated delta rule, KDA, comba) against the
oracle's gradients (reverse mode through the token recurrences): head dims x grouping x packing x in-kernel prologues x
initial state x form of the scans.  The hand-picked matrices of the operators' own test files cover each option; this file
covers their combinations.  Bars: the reference's widest per gradient (tests/ops/test_gdn.py, test_kda.py, test_comba.py)."""
import random

import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu
TOL = dict(dq=0.008, dk=0.008, dv=0.008, dp=0.008, dg=0.02, dbeta=0.02, dh0=0.008)


def _case(seed):
    rnd = random.Random(1000 + seed)
    op = ['gdn', 'kda', 'comba'][seed % 3]
    H, G = rnd.choice([1, 2, 3]), rnd.choice([1, 2])
    K = rnd.choice([24, 64, 100, 128] + ([192, 256] if op == 'gdn' else []))
    V = rnd.choice([32, 64, 128, 160])
    packed = rnd.random() < 0.4
    if packed:
        lens = [rnd.choice([1, 63, 64, 65, 130, 200]) for _ in range(rnd.choice([1, 2, 4]))]
        cu = [0]
        for x in lens:
            cu.append(cu[-1] + x)
        B, T, N = 1, cu[-1], len(lens)
    else:
        B = rnd.choice([1, 2])
        T, cu, N = rnd.choice([1, 64, 129, 300, 520]), None, B
    return dict(op=op, H=H, HV=H * G, K=K, V=V, B=B, T=T, N=N, cu=cu, dtype=rnd.choice([torch.bfloat16, torch.float16]),
                l2=rnd.random() < 0.5, gate=op != 'comba' and rnd.random() < 0.4, sig=op != 'comba' and rnd.random() < 0.4,
                h0=rnd.random() < 0.7, dht=rnd.random() < 0.7, scale=rnd.choice([None, 0.1, 1.0]),
                vfirst=op != 'comba' and rnd.random() < 0.3, mode=rnd.choice(['auto', 'segments', 'wide']))


@pytest.mark.parametrize('seed', range(96))
def test_random_backward(seed, monkeypatch):
    c = _case(seed)
    op, B, T, H, HV, K, V, N, cu, dtype = (c[n] for n in ('op', 'B', 'T', 'H', 'HV', 'K', 'V', 'N', 'cu', 'dtype'))
    gen = torch.Generator().manual_seed(seed)
    q, k, p = (torch.randn(B, T, H, K, generator=gen) for _ in range(3))
    if not c['l2']:
        q, k, p = (F.normalize(x, dim=-1) for x in (q, k, p))
    q, k, p = q.to(dtype), k.to(dtype), p.to(dtype)
    v = torch.randn(B, T, HV, V, generator=gen).to(dtype)
    gshape = (B, T, HV, K) if op == 'kda' else (B, T, HV)
    g = torch.randn(*gshape, generator=gen)
    A_log = dt_bias = None
    if c['gate']:
        A_log = 0.3 * torch.randn(HV, generator=gen)
        dt_bias = 0.3 * torch.randn(HV * K if op == 'kda' else HV, generator=gen)
    else:
        g = F.logsigmoid(g) / 2
    beta = torch.randn(B, T, HV, generator=gen) if c['sig'] else torch.rand(B, T, HV, generator=gen)
    sshape = (N, HV, V, K) if c['vfirst'] else (N, HV, K, V)
    h0 = 0.5 * torch.randn(*sshape, generator=gen) if c['h0'] else None
    dht = torch.randn(*sshape, generator=gen) if c['dht'] else None
    do = torch.randn(B, T, HV, V, generator=gen).to(dtype)
    kw = dict(scale=c['scale'], use_qk_l2norm_in_kernel=c['l2'])
    if op != 'comba':
        kw.update(use_gate_in_kernel=c['gate'], use_beta_sigmoid_in_kernel=c['sig'], state_v_first=c['vfirst'])
    monkeypatch.setenv('FLA_HIP_BWD_SCAN_MODE', c['mode'])
    dev = lambda x: None if x is None else x.cuda().requires_grad_(True)
    cu_t = None if cu is None else torch.tensor(cu, device='cuda')
    if op == 'gdn':
        from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
        ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, A_log=A_log, dt_bias=dt_bias,
                                       dtype=torch.float32, **kw)
        leaves = dict(dq=dev(q), dk=dev(k), dv=dev(v), dg=dev(g), dbeta=dev(beta), dh0=dev(h0), dA_log=dev(A_log), ddt_bias=dev(dt_bias))
        o, ht = chunk_gated_delta_rule(leaves['dq'], leaves['dk'], leaves['dv'], leaves['dg'], leaves['dbeta'], initial_state=leaves['dh0'],
                                       output_final_state=True, cu_seqlens=cu_t, A_log=leaves['dA_log'], dt_bias=leaves['ddt_bias'], **kw)
    elif op == 'kda':
        from fla_hip.ops.kda import chunk_kda
        ref = O.kda_grads(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, A_log=A_log, dt_bias=dt_bias, dtype=torch.float32, **kw)
        leaves = dict(dq=dev(q), dk=dev(k), dv=dev(v), dg=dev(g), dbeta=dev(beta), dh0=dev(h0), dA_log=dev(A_log), ddt_bias=dev(dt_bias))
        o, ht = chunk_kda(leaves['dq'], leaves['dk'], leaves['dv'], leaves['dg'], leaves['dbeta'], initial_state=leaves['dh0'],
                          output_final_state=True, cu_seqlens=cu_t, A_log=leaves['dA_log'], dt_bias=leaves['ddt_bias'], **kw)
    else:
        from fla_hip.ops.comba import chunk_comba
        ref = O.comba_grads(q, k, v, p, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, dtype=torch.float32, **kw)
        leaves = dict(dq=dev(q), dk=dev(k), dv=dev(v), dp=dev(p), dg=dev(g), dbeta=dev(beta), dh0=dev(h0))
        o, ht = chunk_comba(leaves['dq'], leaves['dk'], leaves['dv'], leaves['dp'], leaves['dg'], leaves['dbeta'], initial_state=leaves['dh0'],
                            output_final_state=True, cu_seqlens=cu_t, **kw)
    loss = (o.float() * do.cuda().float()).sum()
    if dht is not None:
        loss = loss + (ht * dht.cuda()).sum()
    loss.backward()
    for n, r in ref.items():
        if r is None:
            continue
        x = leaves[n].grad.float().cpu()
        assert x.shape == r.shape and not torch.isnan(x).any(), (c, n)
        if O.get_abs_err(r, x) <= 1e-6:             # (fla/utils/_testing.py:28-34: gradients that vanish)
            continue
        if not r.any() and O.get_abs_err(r, x) <= 1e-5:
            continue    # exactly zero in the oracle (one token on an empty state: dg); the kernels cancel fp32 terms of order ten
        if n in ('dA_log', 'ddt_bias'):
            # each entry sums the gate's gradient over every token (ddt_bias exactly so, dA_log with weights above one): terms of
            # both signs, so the error is measured against the size of what is summed, not of what is left
            e = float((x - r).abs().max() / (ref['dg'].abs().sum() / r.numel()))
            assert e <= TOL['dg'], f'{c}: {n} error {e:.3e} of the summed |dg| > {TOL["dg"]}'
            continue
        e = O.get_err_ratio(r, x)
        assert e <= TOL[n], f'{c}: {n} rel-rmse {e:.3e} > {TOL[n]}'
