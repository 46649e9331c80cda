"""Seeded random combinations of shapes, layouts and switches for both operators against the CPU oracle: the
hand-picked matrices of the other test files cover each option; this file covers their combinations (head dims x
grouping x packing x state layout x in-kernel prologues x form of the sequential stage)."""
import random

import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu
DEV = 'cuda'


def _case(seed, recurrent):
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.bfloat16, torch.float16] + ([torch.float32] if recurrent else []))
    H = rnd.choice([1, 2, 3])
    G = rnd.choice([1, 2, 4])
    if recurrent:
        K, V = rnd.choice([16, 32, 64, 100, 128, 192, 256]), rnd.choice([16, 40, 64, 128, 200])
    else:
        K, V = rnd.choice([8, 24, 60, 64, 96, 100, 128]), rnd.choice([16, 56, 64, 100, 128, 160])
    packed = rnd.random() < 0.5
    if packed:
        n = rnd.choice([1, 2, 3, 5])
        lens = [rnd.choice([1, 7, 63, 64, 65, 130, 200]) for _ in range(n)]
        if recurrent:
            lens = [min(x, 40) for x in lens]
        cu = [0]
        for x in lens:
            cu.append(cu[-1] + x)
        B, T, N = 1, cu[-1], n
    else:
        B, N = rnd.choice([1, 2, 3]), None
        T = rnd.choice([1, 5, 33] if recurrent else [1, 63, 64, 129, 300, 700])
        cu, N = None, B
    flags = dict(l2=rnd.random() < 0.5, gate=rnd.random() < 0.4, sig=rnd.random() < 0.4, neg=False,
                 vfirst=rnd.random() < 0.5, h0=rnd.random() < 0.7, scale=rnd.choice([None, 0.1, 1.0]))
    flags['neg'] = flags['sig'] and rnd.random() < 0.5
    mode = rnd.choice(['auto', 'wide-single', 'wide-pair', 'segments-single', 'segments-pair', 'segments-exact-single'])
    return dict(dtype=dtype, H=H, HV=H * G, K=K, V=V, B=B, T=T, N=N, cu=cu, mode=mode, **flags)


def _inputs(c, seed):
    gen = torch.Generator().manual_seed(seed)
    B, T, H, HV, K, V = c['B'], c['T'], c['H'], c['HV'], c['K'], c['V']
    q, k = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen)
    if not c['l2']:
        q, k = F.normalize(q, dim=-1), F.normalize(k, dim=-1)
    q, k = q.to(c['dtype']), k.to(c['dtype'])
    v = torch.randn(B, T, HV, V, generator=gen).to(c['dtype'])
    g = torch.randn(B, T, HV, generator=gen)
    beta = torch.randn(B, T, HV, generator=gen)
    A_log = dt_bias = None
    if c['gate']:
        A_log, dt_bias = 0.3 * torch.randn(HV, generator=gen), 0.3 * torch.randn(HV, generator=gen)
    else:
        g = F.logsigmoid(g) / 4
    if not c['sig']:
        beta = torch.sigmoid(beta)
    h0 = 0.5 * torch.randn(c['N'], HV, K, V, generator=gen) if c['h0'] else None
    return q, k, v, g, beta, A_log, dt_bias, h0


def _compare(c, ref, got, tol):
    for name, r, x in zip(('o', 'ht'), ref, got):
        x = x.float().cpu()
        if name == 'ht' and c['vfirst']:
            x = x.transpose(-1, -2)
        assert x.shape == r.shape, (name, x.shape, r.shape)
        assert not torch.isnan(x).any(), f'{name}: NaN in {c}'
        err, m = O.get_err_ratio(r, x), O.max_abs_ratio(r, x)
        assert err <= tol and m <= 2 * tol, f'{name}: rel-rmse {err:.2e} max-abs {m:.2e} for {c}'


@pytest.mark.parametrize('seed', list(range(48)) + [f'wide{i}' for i in range(24)])
def test_chunk_random_configuration(seed, monkeypatch):
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    if isinstance(seed, str):
        # the same combinations with wide keys (128 < K <= 256) and any number of value columns
        seed = 500 + int(seed[4:])
        c = _case(seed, recurrent=False)
        rnd = random.Random(seed + 7)
        c['K'], c['V'] = rnd.choice([136, 160, 192, 250, 256]), rnd.choice([16, 64, 72, 128, 200, 320])
    else:
        c = _case(seed, recurrent=False)
    if c['mode'] != 'auto':
        monkeypatch.setenv('FLA_HIP_SCAN_MODE', c['mode'])
    q, k, v, g, beta, A_log, dt_bias, h0 = _inputs(c, 1000 + seed)
    kw = dict(use_qk_l2norm_in_kernel=c['l2'], use_gate_in_kernel=c['gate'], use_beta_sigmoid_in_kernel=c['sig'],
              allow_neg_eigval=c['neg'])
    ref = O.chunk_gated_delta_rule(q, k, v, g, beta, c['scale'], h0, True, cu_seqlens=c['cu'], A_log=A_log, dt_bias=dt_bias, **kw)
    d = lambda t: None if t is None else t.to(DEV)
    h0d = None if h0 is None else (h0.transpose(-1, -2).contiguous() if c['vfirst'] else h0).to(DEV)
    got = chunk_gated_delta_rule(d(q), d(k), d(v), d(g), d(beta), scale=c['scale'], initial_state=h0d, output_final_state=True,
                                 state_v_first=c['vfirst'], A_log=d(A_log), dt_bias=d(dt_bias),
                                 cu_seqlens=None if c['cu'] is None else torch.tensor(c['cu'], device=DEV), **kw)
    _compare(c, ref, got, 5e-3)


@pytest.mark.parametrize('seed', range(48))
def test_recurrent_random_configuration(seed):
    from fla_hip.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    c = _case(seed, recurrent=True)
    q, k, v, g, beta, A_log, dt_bias, h0 = _inputs(c, 2000 + seed)
    kw = dict(use_qk_l2norm_in_kernel=c['l2'], use_gate_in_kernel=c['gate'], use_beta_sigmoid_in_kernel=c['sig'],
              allow_neg_eigval=c['neg'])
    ref = O.recurrent_gated_delta_rule(q, k, v, g, beta, c['scale'], h0, True, cu_seqlens=c['cu'], A_log=A_log, dt_bias=dt_bias, **kw)
    d = lambda t: None if t is None else t.to(DEV)
    h0d = None if h0 is None else (h0.transpose(-1, -2).contiguous() if c['vfirst'] else h0).to(DEV)
    got = fused_recurrent_gated_delta_rule(d(q), d(k), d(v), d(g), beta=d(beta), scale=c['scale'], initial_state=h0d,
                                           output_final_state=True, state_v_first=c['vfirst'], A_log=d(A_log), dt_bias=d(dt_bias),
                                           cu_seqlens=None if c['cu'] is None else torch.tensor(c['cu'], device=DEV), **kw)
    _compare(c, ref, got, 2e-3 if c['dtype'] == torch.float32 else 5e-3)
