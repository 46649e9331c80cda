"""Backward of chunk_gated_delta_rule.

CPU part: the oracle's gradients (reverse-mode differentiation of the token recurrence) are pinned by central
finite differences of the recurrence itself, and the stage-by-stage restatement of the reference's chunked
backward pass is pinned against those gradients.
GPU part: gradients from the HIP kernels (autograd through the product's operator, C ABI underneath) against
the oracle's on the same seeded inputs; cases and tolerances follow the reference's tests
(tests/ops/test_gdn.py:108-200 dq, dk, dv, dh0 0.008, dbeta, dg 0.02; :281-370; :712-803 packed sequences)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

TOL = dict(dq=0.008, dk=0.008, dv=0.008, dbeta=0.02, dg=0.02, dh0=0.008)


# --------------------------------------------------------------------------------------------
# oracle pins (CPU)
# --------------------------------------------------------------------------------------------
def _loss(q, k, v, g, beta, h0, do, dht, **kw):
    o, ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                         dtype=torch.float64, **kw)
    return float((o * do).sum() + (ht * dht).sum())


@pytest.mark.parametrize('kw', [
    dict(),
    dict(use_qk_l2norm_in_kernel=True),
    dict(use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True),
    dict(use_gate_in_kernel=True),
    dict(cu_seqlens=[0, 5, 12]),
    dict(state_v_first=True),
])
def test_oracle_grads_match_finite_differences(kw):
    B, T, H, HV, K, V = (1, 12, 2, 4, 6, 5) if 'cu_seqlens' in kw else (2, 9, 2, 4, 6, 5)
    N = 2
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, K, V, seed=7, h0_std=0.5, N=N, dtype=torch.float64)
    q, k = q * 1.7, k * 0.8                              # not unit rows: the l2 norm must matter
    gen = torch.Generator().manual_seed(8)
    g, beta = g.double(), beta.double()
    A_log = dt_bias = None
    if kw.get('use_gate_in_kernel'):
        g = torch.randn(B, T, HV, generator=gen, dtype=torch.float64)
        A_log = torch.randn(HV, generator=gen, dtype=torch.float64) * 0.3
        dt_bias = torch.randn(HV, generator=gen, dtype=torch.float64) * 0.3
        kw = dict(kw, A_log=A_log, dt_bias=dt_bias)
    if kw.get('use_beta_sigmoid_in_kernel'):
        beta = torch.randn(B, T, HV, generator=gen, dtype=torch.float64)
    h0 = h0.double()
    if kw.get('state_v_first'):
        h0 = h0.transpose(-1, -2).contiguous()
    do = torch.randn(B, T, HV, V, generator=gen, dtype=torch.float64)
    dht = torch.randn(*h0.shape, generator=gen, dtype=torch.float64)
    grads = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, **kw)
    inputs = dict(dq=q, dk=k, dv=v, dg=g, dbeta=beta, dh0=h0)
    if A_log is not None:
        inputs.update(dA_log=A_log, ddt_bias=dt_bias)
    eps = 1e-6
    for name, x in inputs.items():
        d = torch.randn(x.shape, generator=gen, dtype=torch.float64)

        def at(step):
            args = {n: (t + step * d if n == name else t) for n, t in inputs.items()}
            kw2 = dict(kw)
            if A_log is not None:
                kw2.update(A_log=args['dA_log'], dt_bias=args['ddt_bias'])
            return _loss(args['dq'], args['dk'], args['dv'], args['dg'], args['dbeta'], args['dh0'], do, dht, **kw2)
        fd = (at(eps) - at(-eps)) / (2 * eps)
        an = float((grads[name] * d).sum())
        assert abs(fd - an) <= 1e-6 * max(1.0, abs(an)), f'{name}: finite difference {fd} vs gradient {an}'


@pytest.mark.parametrize('T,HV,K,V,C', [(150, 2, 16, 24, 64), (64, 1, 8, 8, 64), (37, 3, 12, 8, 16), (100, 2, 8, 8, 32)])
def test_oracle_chunked_backward_matches_recurrence_grads(T, HV, K, V, C):
    q, k, v, g, beta, h0 = O.make_inputs(1, T, HV, HV, K, V, seed=T, h0_std=0.5, dtype=torch.float64)
    gen = torch.Generator().manual_seed(T + 1)
    do = torch.randn(1, T, HV, V, generator=gen, dtype=torch.float64)
    dht = torch.randn(1, HV, K, V, generator=gen, dtype=torch.float64)
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, scale=0.3, initial_state=h0)
    got = O.chunk_backward_one_sequence(q[0], k[0], v[0], g[0], beta[0], 0.3, h0[0], do[0], dht[0], chunk_size=C)
    for n in TOL:
        assert O.get_err_ratio(ref[n][0], got[n]) < 1e-12, n


# --------------------------------------------------------------------------------------------
# HIP kernels against the oracle (GPU)
# --------------------------------------------------------------------------------------------
def _op():
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    return chunk_gated_delta_rule


def _grads_gpu(q, k, v, g, beta, h0, do, dht, cu=None, **kw):
    dev = 'cuda'
    leaves = {n: (None if x is None else x.to(dev).requires_grad_(True))
              for n, x in dict(dq=q, dk=k, dv=v, dg=g, dbeta=beta, dh0=h0).items()}
    extra = {}
    for n in ('A_log', 'dt_bias'):
        if kw.get(n) is not None:
            extra['d' + n] = kw[n] = kw[n].to(dev).requires_grad_(True)
    cu_t = None if cu is None else torch.tensor(cu, dtype=kw.pop('idx_dtype', torch.int64), device=dev)
    o, ht = _op()(leaves['dq'], leaves['dk'], leaves['dv'], leaves['dg'], leaves['dbeta'], initial_state=leaves['dh0'],
                  output_final_state=dht is not None, cu_seqlens=cu_t, **kw)
    loss = (o.float() * do.to(dev).float()).sum()
    if dht is not None:
        loss = loss + (ht * dht.to(dev)).sum()
    loss.backward()
    out = {n: (None if x is None else x.grad) for n, x in leaves.items()}
    out.update({n: x.grad for n, x in extra.items()})
    return o, ht, out


def _compare(ref, got, tol=TOL, names=None):
    for n in names or [n for n in ref if ref[n] is not None]:
        x = got[n].detach().float().cpu()
        assert x.shape == ref[n].shape, f'{n}: shape {tuple(x.shape)} vs {tuple(ref[n].shape)}'
        assert not torch.isnan(x).any(), f'{n}: NaN'
        if O.get_abs_err(ref[n], x) <= 1e-6:       # (fla/utils/_testing.py:28-34: gradients that vanish, e.g. dg under extreme decay)
            continue
        r = O.get_err_ratio(ref[n], x)
        assert r <= tol.get(n, 0.02), f'{n}: rel-rmse {r:.3e} > {tol.get(n, 0.02)}'


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,HV,D,scale,gate_div,mask_p,l2,dtype', [
    (1, 64, 1, 1, 128, None, 1.0, 0, False, torch.bfloat16),
    (2, 75, 4, 4, 64, 1, 0.01, 0, False, torch.float16),          # the reference's matrix (shorter where it is long)
    (2, 500, 3, 3, 60, 1, 1, 0, False, torch.float16),
    (2, 300, 3, 3, 64, 0.1, 1, 0.5, False, torch.float16),
    (1, 512, 4, 4, 100, 1, 0.1, 0, False, torch.float16),
    (2, 256, 4, 4, 128, 0.1, 1, 1.0, False, torch.float16),
    (2, 512, 4, 4, 128, 0.1, 1, 0, True, torch.float16),
    (1, 700, 4, 4, 128, 0.1, 10, 0, False, torch.float16),
    (2, 256, 2, 4, 64, 1, 1, 0, False, torch.float16),
    (2, 512, 2, 8, 64, 1, 0.1, 0, True, torch.float16),
    (2, 200, 2, 4, 128, None, 4.0, 0, False, torch.bfloat16),
    (1, 130, 2, 2, 128, None, 4.0, 0, True, torch.bfloat16),
    (3, 100, 12, 24, 128, None, 4.0, 0, True, torch.bfloat16),       # 72 runs: the two scans apart, 128 value columns per workgroup
    (2, 70, 80, 80, 128, None, 4.0, 0, False, torch.bfloat16),       # 160 runs: one scan after the other, 128 columns
    (2, 130, 20, 20, 128, None, 4.0, 0, True, torch.bfloat16),       # 40 runs: apart at 64 columns; the l2 norm inside the kernels
    (1, 100, 72, 72, 100, None, 4.0, 0, True, torch.float16),        # 72 runs apart at 128 columns, the l2 norm inside, K padded
])
def test_chunk_backward(B, T, H, HV, D, scale, gate_div, mask_p, l2, dtype):
    gen = torch.Generator().manual_seed(42)
    q = torch.rand(B, T, H, D, generator=gen)
    k = torch.rand(B, T, H, D, generator=gen)
    if not l2:
        q, k = F.normalize(q, p=2, dim=-1), F.normalize(k, p=2, dim=-1)
    q, k = q.to(dtype), k.to(dtype)
    v = torch.rand(B, T, HV, D, generator=gen).to(dtype)
    beta = torch.rand(B, T, HV, generator=gen).sigmoid()
    g = F.logsigmoid(torch.rand(B, T, HV, generator=gen)) / gate_div
    g = g * (torch.rand(B, T, HV, generator=gen) > mask_p)
    h0 = torch.randn(B, HV, D, D, generator=gen) * 0.3
    do = torch.randn(B, T, HV, D, generator=gen).to(dtype)
    dht = torch.randn(B, HV, D, D, generator=gen)
    kw = dict(scale=scale, use_qk_l2norm_in_kernel=l2)
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, dtype=torch.float32, **kw)
    o, ht, got = _grads_gpu(q, k, v, g, beta, h0, do, dht, **kw)
    assert got['dq'].dtype == dtype and got['dv'].dtype == dtype and got['dg'].dtype == g.dtype
    _compare(ref, got)


@pytest.mark.gpu
@pytest.mark.parametrize('H,HV,D,mask_p,cu', [
    (4, 4, 60, 0, [0, 15]),
    (4, 4, 64, 0, [0, 256, 500, 1000]),
    (4, 4, 64, 0.5, [0, 256, 500, 1000]),
    (2, 2, 100, 0, [0, 15, 100, 300, 700]),
    (2, 4, 64, 0, [0, 256, 500, 1000]),
    (2, 8, 128, 0, [0, 1, 65, 200, 264]),
])
def test_chunk_backward_packed(H, HV, D, mask_p, cu):
    gen = torch.Generator().manual_seed(42)
    T, N = cu[-1], len(cu) - 1
    dtype = torch.float16
    q = torch.randn(1, T, H, D, generator=gen).to(dtype)
    k = F.normalize(torch.randn(1, T, H, D, generator=gen), p=2, dim=-1).to(dtype)
    v = torch.randn(1, T, HV, D, generator=gen).to(dtype)
    g = F.logsigmoid(torch.rand(1, T, HV, generator=gen))
    g = g * (torch.rand(1, T, HV, generator=gen) > mask_p)
    beta = torch.rand(1, T, HV, generator=gen).sigmoid()
    h0 = torch.randn(N, HV, D, D, generator=gen)
    do = torch.randn(1, T, HV, D, generator=gen).to(dtype)
    dht = torch.rand(N, HV, D, D, generator=gen)
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, dtype=torch.float32)
    o, ht, got = _grads_gpu(q, k, v, g, beta, h0, do, dht, cu=cu, idx_dtype=torch.int32 if D == 64 else torch.int64)
    _compare(ref, got, tol=dict(dq=0.007, dk=0.008, dv=0.007, dbeta=0.015, dg=0.015, dh0=0.007))
    # every sequence's gradients are those of the sequence alone
    if N > 1:
        s, e = cu[1], cu[2]
        _, _, alone = _grads_gpu(q[:, s:e], k[:, s:e], v[:, s:e], g[:, s:e], beta[:, s:e], h0[1:2], do[:, s:e], dht[1:2])
        for n in ('dq', 'dk', 'dv'):
            assert O.get_err_ratio(got[n][:, s:e].float().cpu(), alone[n].float().cpu()) < 2e-3, n


@pytest.mark.gpu
def test_chunk_backward_packed_tokens_outside_every_sequence_get_zero_gradients():
    # boundaries that start after token 0 and end before the last one: the padding tokens belong to no sequence, the
    # kernels never write them, and what autograd hands on for them must be zero (not whatever the allocator held)
    cu, T, H, HV, D = [70, 200, 390], 460, 2, 4, 64
    gen = torch.Generator().manual_seed(5)
    q, k, v, g, beta, h0 = O.make_inputs(1, T, H, HV, D, D, seed=5, h0_std=0.5, N=2, dtype=torch.bfloat16)
    do = torch.randn(1, T, HV, D, generator=gen).bfloat16()
    dht = torch.randn(2, HV, D, D, generator=gen)
    # poison the caching allocator's free blocks so that an uninitialised buffer would show
    junk = [torch.full((1, T, HV, D), float('nan'), device='cuda', dtype=dt) for dt in (torch.bfloat16, torch.float32) for _ in range(4)]
    del junk
    _, _, got = _grads_gpu(q, k, v, g, beta, h0, do, dht, cu=cu)
    for n in ('dq', 'dk', 'dv', 'dg', 'dbeta'):
        x = got[n].float().cpu()
        assert not torch.isnan(x).any(), n
        assert not x[:, :cu[0]].any() and not x[:, cu[-1]:].any(), f'{n}: tokens outside the sequences'
    sl = slice(cu[0], cu[-1])
    ref = O.gated_delta_rule_grads(q[:, sl], k[:, sl], v[:, sl], g[:, sl], beta[:, sl], do[:, sl], dht, initial_state=h0,
                                   cu_seqlens=[c - cu[0] for c in cu], dtype=torch.float32)
    _compare(ref, {n: (x[:, sl] if n != 'dh0' else x) for n, x in got.items()})


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,HV,K,V,l2,cu', [
    (2, 200, 2, 4, 256, 128, True, None),
    (1, 130, 2, 2, 256, 256, False, None),
    (1, 300, 1, 2, 192, 128, True, None),
    (1, 257, 2, 2, 256, 512, True, None),                  # the reference layer's default head shape (head_dim 256, expand_v 2)
    (1, 0, 2, 4, 160, 64, False, [0, 100, 101, 300]),
    (3, 100, 12, 24, 256, 128, True, None),                 # 72 runs: the forward scan takes 64 columns per workgroup
    (2, 130, 16, 32, 256, 256, False, None),                # 128 runs: the reverse scan takes 64 columns, P^T straight from memory
    (1, 70, 136, 136, 200, 64, True, None),                 # 136 runs, a ragged chunk
])
def test_chunk_backward_wide_keys(B, T, H, HV, K, V, l2, cu):
    """Key head dims above 128 (two blocks of 128 key features in every backward kernel)."""
    if cu is not None:
        T = cu[-1]
    N = B if cu is None else len(cu) - 1
    gen = torch.Generator().manual_seed(5)
    q, k = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen)
    if not l2:
        q, k = F.normalize(q, p=2, dim=-1), F.normalize(k, p=2, dim=-1)
    q, k = q.bfloat16(), k.bfloat16()
    v = torch.randn(B, T, HV, V, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, HV, generator=gen)) / 4
    beta = torch.rand(B, T, HV, generator=gen).sigmoid()
    h0 = torch.randn(N, HV, K, V, generator=gen) * 0.3
    do = torch.randn(B, T, HV, V, generator=gen).bfloat16()
    dht = torch.randn(N, HV, K, V, generator=gen)
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, use_qk_l2norm_in_kernel=l2,
                                   dtype=torch.float32)
    o, ht, got = _grads_gpu(q, k, v, g, beta, h0, do, dht, cu=cu, use_qk_l2norm_in_kernel=l2)
    _compare(ref, got)


@pytest.mark.gpu
@pytest.mark.parametrize('what', ['beta_sigmoid', 'beta_sigmoid_neg', 'gate', 'gate_no_bias', 'v_first', 'no_h0', 'no_dht',
                                  'wide_v', 'fp32'])
def test_chunk_backward_options(what):
    B, T, H, HV, D = 2, 200, 2, 4, 128
    V = 256 if what == 'wide_v' else D
    dtype = torch.float32 if what == 'fp32' else torch.bfloat16
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, D, V, seed=11, gate_div=4.0, h0_std=0.3, dtype=dtype)
    gen = torch.Generator().manual_seed(12)
    do = torch.randn(B, T, HV, V, generator=gen).to(dtype)
    dht = torch.randn(B, HV, D, V, generator=gen)
    kw = {}
    if what.startswith('beta_sigmoid'):
        beta = torch.randn(B, T, HV, generator=gen)
        kw = dict(use_beta_sigmoid_in_kernel=True, allow_neg_eigval=what.endswith('neg'))
    if what.startswith('gate'):
        g = torch.randn(B, T, HV, generator=gen)
        kw = dict(use_gate_in_kernel=True, A_log=torch.randn(HV, generator=gen) * 0.5,
                  dt_bias=None if what == 'gate_no_bias' else torch.randn(HV, generator=gen) * 0.5)
    if what == 'v_first':
        h0, dht = h0.transpose(-1, -2).contiguous(), dht.transpose(-1, -2).contiguous()
        kw = dict(state_v_first=True)
    if what == 'no_h0':
        h0 = None
    if what == 'no_dht':
        dht = None
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, dtype=torch.float32,
                                   **{n: x for n, x in kw.items()})
    o, ht, got = _grads_gpu(q, k, v, g, beta, h0, do, dht, **dict(kw))
    _compare(ref, got)


@pytest.mark.gpu
@pytest.mark.parametrize('seed', range(24))
def test_chunk_backward_random(seed):
    """Seeded random combinations of head dims, grouping, packing, state layout, prologues and dtype."""
    import random
    rnd = random.Random(1000 + seed)
    D = rnd.choice([16, 32, 40, 64, 96, 128])
    V = rnd.choice([D, 64, 128, 192]) if seed % 4 == 0 else D
    H = rnd.choice([1, 2, 3])
    HV = H * rnd.choice([1, 1, 2, 4])
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    packed = rnd.random() < 0.4
    if packed:
        N = rnd.randint(1, 4)
        cu = [0]
        for _ in range(N):
            cu.append(cu[-1] + rnd.choice([1, 7, 63, 64, 65, 130, 200]))
        B, T = 1, cu[-1]
    else:
        B, T, cu = rnd.randint(1, 3), rnd.choice([1, 5, 64, 100, 129, 257]), None
        N = B
    kw = {}
    gen = torch.Generator().manual_seed(2000 + seed)
    q, k = torch.randn(B, T, H, D, generator=gen), torch.randn(B, T, H, D, generator=gen)
    if rnd.random() < 0.5:
        kw['use_qk_l2norm_in_kernel'] = True
    else:
        q, k = F.normalize(q, p=2, dim=-1), F.normalize(k, p=2, dim=-1)
    q, k = q.to(dtype), k.to(dtype)
    v = torch.randn(B, T, HV, V, generator=gen).to(dtype)
    g = F.logsigmoid(torch.randn(B, T, HV, generator=gen)) / rnd.choice([1.0, 4.0, 16.0])
    beta = torch.rand(B, T, HV, generator=gen).sigmoid()
    if rnd.random() < 0.3:
        beta = torch.randn(B, T, HV, generator=gen)
        kw.update(use_beta_sigmoid_in_kernel=True, allow_neg_eigval=rnd.random() < 0.5)
    if rnd.random() < 0.3:
        g = torch.randn(B, T, HV, generator=gen)
        kw.update(use_gate_in_kernel=True, A_log=torch.randn(HV, generator=gen) * 0.5,
                  dt_bias=torch.randn(HV, generator=gen) * 0.5 if rnd.random() < 0.5 else None)
    vfirst = rnd.random() < 0.3
    h0 = torch.randn(N, HV, D, V, generator=gen) * 0.3 if rnd.random() < 0.7 else None
    dht = torch.randn(N, HV, D, V, generator=gen) if rnd.random() < 0.7 else None
    if vfirst:
        kw['state_v_first'] = True
        h0 = None if h0 is None else h0.transpose(-1, -2).contiguous()
        dht = None if dht is None else dht.transpose(-1, -2).contiguous()
    do = torch.randn(B, T, HV, V, generator=gen).to(dtype)
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, dtype=torch.float32, **kw)
    o, ht, got = _grads_gpu(q, k, v, g, beta, h0, do, dht, cu=cu, **dict(kw))
    # (single tokens and very short sequences: the rounding of a handful of bf16 products is all there is to compare)
    tol = TOL if T >= 64 else {n: 2 * x for n, x in TOL.items()}
    _compare(ref, got, tol=tol)


@pytest.mark.gpu
def test_chunk_backward_empty_sequences_and_no_tokens():
    """Packed input with sequences of length zero: their dh0 is their dht, nobody else's gradient moves."""
    H, D = 2, 128
    cu = [0, 0, 70, 70, 134]
    T, N = cu[-1], len(cu) - 1
    gen = torch.Generator().manual_seed(3)
    q, k, v, g, beta, _ = O.make_inputs(1, T, H, H, D, D, seed=3, gate_div=4.0, dtype=torch.bfloat16)
    h0 = torch.randn(N, H, D, D, generator=gen) * 0.3
    do = torch.randn(1, T, H, D, generator=gen).bfloat16()
    dht = torch.randn(N, H, D, D, generator=gen)
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, dtype=torch.float32)
    o, ht, got = _grads_gpu(q, k, v, g, beta, h0, do, dht, cu=cu)
    _compare(ref, got)
    assert torch.equal(got['dh0'][0].cpu(), dht[0]) and torch.equal(got['dh0'][2].cpu(), dht[2])
    # no token at all
    e = torch.zeros(1, 0, H, D, dtype=torch.bfloat16)
    z = torch.zeros(1, 0, H)
    o, ht, got = _grads_gpu(e, e, e, z, z, h0[:1], e, dht[:1])
    assert o.shape == (1, 0, H, D) and torch.equal(got['dh0'].cpu(), dht[:1]) and got['dq'].shape == e.shape


@pytest.mark.gpu
def test_chunk_backward_full_size_properties():
    """At the size of a published shape (B=1 T=8192 H=32 of 96, D=128) the CPU oracle is out of reach; what the algebra fixes is not:
    two runs give the same bits, gradients are linear in (do, dht) - doubling both doubles every gradient bit for bit - and a sequence cut in two,
    chained through the state forward and through its gradient backward, gives the gradients of the whole."""
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    dev = 'cuda'
    B, T, H, D = 1, 8192, 32, 128
    gen = torch.Generator().manual_seed(9)
    q = F.normalize(torch.randn(B, T, H, D, generator=gen), dim=-1).bfloat16().to(dev)
    k = F.normalize(torch.randn(B, T, H, D, generator=gen), dim=-1).bfloat16().to(dev)
    v = torch.randn(B, T, H, D, generator=gen).bfloat16().to(dev)
    g = (F.logsigmoid(torch.randn(B, T, H, generator=gen)) / 4).to(dev)
    beta = torch.rand(B, T, H, generator=gen).sigmoid().to(dev)
    h0 = (torch.randn(B, H, D, D, generator=gen) * 0.3).to(dev)
    do = torch.randn(B, T, H, D, generator=gen).bfloat16().to(dev)
    dht = torch.randn(B, H, D, D, generator=gen).to(dev)

    def grads(sl, h_in, do_, dht_):
        xs = [x[:, sl].detach().clone().requires_grad_(True) for x in (q, k, v, g, beta)] + [h_in.detach().clone().requires_grad_(True)]
        o, ht = chunk_gated_delta_rule(*xs[:5], initial_state=xs[5], output_final_state=True)
        ((o.float() * do_[:, sl].float()).sum() + (ht * dht_).sum()).backward()
        return [x.grad for x in xs], ht.detach()

    whole, _ = grads(slice(0, T), h0, do, dht)
    again, _ = grads(slice(0, T), h0, do, dht)
    twice, _ = grads(slice(0, T), h0, do * 2, dht * 2)
    for name, a, b, c in zip(('dq', 'dk', 'dv', 'dg', 'dbeta', 'dh0'), whole, twice, again):
        assert torch.equal(a, c), f'{name}: two runs differ'
        assert torch.equal((a.float() * 2).to(a.dtype), b), f'{name}: not linear in (do, dht)'
    cut = 4096 + 64 * 3
    _, h_mid = grads(slice(0, cut), h0, do, torch.zeros_like(dht))
    second, _ = grads(slice(cut, T), h_mid, do, dht)
    first, _ = grads(slice(0, cut), h0, do, second[5])
    for i, name in enumerate(('dq', 'dk', 'dv', 'dg', 'dbeta')):
        joined = torch.cat([first[i], second[i]], dim=1)
        r = O.get_err_ratio(whole[i].float().cpu(), joined.float().cpu())
        assert r < 4e-3, f'{name}: {r:.3e}'
    assert O.get_err_ratio(whole[5].cpu(), first[5].cpu()) < 4e-3


@pytest.mark.gpu
def test_chunk_backward_c_entry_checks():
    from fla_hip import _lib
    lib = _lib.load()
    assert lib.gdn_chunk_bwd_workspace_bytes(4, 2, 128) > 0 and lib.gdn_chunk_bwd_workspace_bytes(4, 2, 256) > lib.gdn_chunk_bwd_workspace_bytes(4, 2, 128)
    assert lib.gdn_chunk_bwd_workspace_bytes(4, 2, 192) == 0
    x = torch.zeros(1, 64, 1, 64, dtype=torch.bfloat16, device='cuda')
    f = torch.zeros(1, 64, 1, device='cuda')
    ws = torch.zeros(lib.gdn_chunk_bwd_workspace_bytes(1, 1, 128), dtype=torch.uint8, device='cuda')
    args = [x.data_ptr()] * 3 + [f.data_ptr()] * 2 + [None, x.data_ptr(), None] + [x.data_ptr()] * 3 + [f.data_ptr()] * 2 + [None]
    rc = lib.gdn_chunk_bwd(*args, None, None, None, ws.data_ptr(), ws.numel(), 1, 64, 1, 1, 64, 64, 1, 1, 1.0,
                           _lib.DTYPE_BF16, _lib.DTYPE_F32, 0, None)
    assert rc == _lib.GDN_ERR_UNSUPPORTED and 'K = 128 or 256' in _lib.last_error()
    with pytest.raises(NotImplementedError):
        from fla_hip.ops.gated_delta_rule.chunk_bwd import chunk_gated_delta_rule_bwd
        w = torch.zeros(1, 64, 1, 264, dtype=torch.bfloat16, device='cuda')
        chunk_gated_delta_rule_bwd(w, w, w, f, f, 1.0, None, w, None)


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,K,cu', [(2, 200, 3, 128, None), (1, 333, 2, 100, [0, 1, 130, 333]), (1, 64, 1, 24, None)])
def test_chunk_backward_l2norm_inside_the_kernels(B, T, H, K, cu):
    """With one value head per q/k head and K <= 128 the l2 normalisation of q and k, forward and back, is taken inside the
    backward's kernels (C entry gdn_chunk_bwd_qk_l2norm): against the separate route (gdn_l2norm_fwd, gdn_chunk_bwd, then
    gdn_l2norm_bwd on its rounded output) and against the oracle's gradients of the rows before normalisation."""
    from fla_hip import _lib
    from fla_hip.ops.gated_delta_rule import chunk_bwd as M
    gen = torch.Generator().manual_seed(5)
    N = B if cu is None else len(cu) - 1
    q, k = (torch.randn(B, T, H, K, generator=gen).bfloat16() for _ in range(2))
    v, do = (torch.randn(B, T, H, 128, generator=gen).bfloat16() for _ in range(2))
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen)) / 2
    beta = torch.rand(B, T, H, generator=gen)
    h0, dht = 0.5 * torch.randn(N, H, K, 128, generator=gen), torch.randn(N, H, K, 128, generator=gen)
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, use_qk_l2norm_in_kernel=True,
                                   dtype=torch.float32)
    cu_t = None if cu is None else torch.tensor(cu, device='cuda')
    rest = (v.cuda(), g.cuda(), beta.cuda(), K ** -0.5, h0.cuda(), do.cuda(), dht.cuda(), False, cu_t, None, None, 64)
    inside = M.chunk_gated_delta_rule_bwd(q.cuda(), k.cuda(), *rest, qk_l2norm=True)
    qn, q_rstd = M.l2norm_fwd(q.cuda())
    kn, k_rstd = M.l2norm_fwd(k.cuda())
    apart = M.chunk_gated_delta_rule_bwd(qn[..., :K], kn[..., :K], *rest, q_rstd, k_rstd)
    for i, name in enumerate(('dq', 'dk')):
        a, b = inside[i], apart[i]
        assert a.shape == b.shape == (B, T, H, K)
        r = O.get_err_ratio(b.float().cpu(), a.float().cpu())
        assert r < 5e-3, f'{name}: inside the kernels against the separate route {r:.3e}'
        e = O.get_err_ratio(ref[name], a.float().cpu())
        assert e <= TOL[name], f'{name}: rel-rmse {e:.3e} against the oracle'
    for i, name in ((2, 'dv'), (3, 'dbeta'), (4, 'dg'), (5, 'dh0')):       # (the normalised rows may differ in their last bit)
        r = O.get_err_ratio(apart[i].float().cpu(), inside[i].float().cpu())
        assert r < 2e-3, f'{name}: {r:.3e}'
    # the entry's refusals: grouped heads, a workspace without room for the normalised rows
    lib = _lib.load()
    assert lib.gdn_chunk_bwd_qk_l2norm_workspace_bytes(1, 2, 128, 64) > lib.gdn_chunk_bwd_workspace_bytes(1, 2, 128)
    assert lib.gdn_chunk_bwd_qk_l2norm_workspace_bytes(1, 2, 256, 64) == 0
    x = torch.zeros(1, 64, 2, 128, dtype=torch.bfloat16, device='cuda')
    x1 = torch.zeros(1, 64, 1, 128, dtype=torch.bfloat16, device='cuda')
    f = torch.zeros(1, 64, 2, device='cuda')
    ws = torch.zeros(lib.gdn_chunk_bwd_qk_l2norm_workspace_bytes(1, 2, 128, 64), dtype=torch.uint8, device='cuda')
    tail = [x.data_ptr(), f.data_ptr(), f.data_ptr(), None, x.data_ptr(), None] + [x.data_ptr()] * 3 + [f.data_ptr()] * 2 + [None]
    dims = lambda h, n: (None, None, None, ws.data_ptr(), n, 1, 64, h, 2, 128, 128, 1, 1, 1.0, _lib.DTYPE_BF16, _lib.DTYPE_F32, 0, None)
    rc = lib.gdn_chunk_bwd_qk_l2norm(x1.data_ptr(), x1.data_ptr(), *tail, *dims(1, ws.numel()))
    assert rc == _lib.GDN_ERR_UNSUPPORTED and 'H == HV' in _lib.last_error()
    rc = lib.gdn_chunk_bwd_qk_l2norm(x.data_ptr(), x.data_ptr(), *tail, *dims(2, lib.gdn_chunk_bwd_workspace_bytes(1, 2, 128)))
    assert rc == _lib.GDN_ERR_WORKSPACE
    assert lib.gdn_chunk_bwd_qk_l2norm(x.data_ptr(), x.data_ptr(), *tail, *dims(2, ws.numel())) == _lib.GDN_OK
    torch.cuda.synchronize()


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,K,V,cu,dtype,with_h0', [
    (1, 400, 2, 128, 128, [0, 64, 64, 129, 400], torch.bfloat16, True),     # an empty sequence, chunk boundaries
    (1, 1, 1, 128, 128, None, torch.bfloat16, True),                          # one token
    (2, 65, 3, 40, 72, None, torch.float16, True),                            # small head dims, one token past a chunk
    (1, 300, 2, 128, 128, [10, 100, 290], torch.bfloat16, False),             # tokens outside every sequence
    (1, 130, 130, 64, 64, None, torch.bfloat16, True),                        # 130 runs: one scan after the other
])
def test_chunk_backward_l2norm_inside_edge_cases(B, T, H, K, V, cu, dtype, with_h0):
    """The route with the l2 normalisation inside the backward's kernels (autograd, use_qk_l2norm_in_kernel, H == HV) on the edges."""
    op = _op()
    gen = torch.Generator().manual_seed(3)
    N = B if cu is None else len(cu) - 1
    q, k = (torch.randn(B, T, H, K, generator=gen).to(dtype) for _ in range(2))
    v, do = (torch.randn(B, T, H, V, generator=gen).to(dtype) for _ in range(2))
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen)) / 2
    beta = torch.rand(B, T, H, generator=gen)
    h0 = 0.5 * torch.randn(N, H, K, V, generator=gen) if with_h0 else None
    dht = torch.randn(N, H, K, V, generator=gen)
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, use_qk_l2norm_in_kernel=True, dtype=torch.float32)
    dev = lambda x: None if x is None else x.cuda().requires_grad_(True)
    leaves = dict(dq=dev(q), dk=dev(k), dv=dev(v), dg=dev(g), dbeta=dev(beta), dh0=dev(h0))
    cu_t = None if cu is None else torch.tensor(cu, device='cuda')
    o, ht = op(leaves['dq'], leaves['dk'], leaves['dv'], leaves['dg'], leaves['dbeta'], initial_state=leaves['dh0'], output_final_state=True,
               cu_seqlens=cu_t, use_qk_l2norm_in_kernel=True)
    ((o.float() * do.cuda().float()).sum() + (ht * dht.cuda()).sum()).backward()
    for n, r in ref.items():
        if r is None or leaves.get(n) is None:
            continue
        x = leaves[n].grad.float().cpu()
        assert x.shape == r.shape and not torch.isnan(x).any(), n
        if O.get_abs_err(r, x) <= 1e-5:             # (gradients that vanish; exactly zero in the oracle: one token on an empty state)
            continue
        e = O.get_err_ratio(r, x)
        assert e <= TOL[n], f'{n}: rel-rmse {e:.3e} > {TOL[n]}'
    if cu is not None and cu[0] > 0:                 # (tokens outside every sequence get zero gradients)
        for n in ('dq', 'dk', 'dv'):
            assert not leaves[n].grad[:, :cu[0]].any() and not leaves[n].grad[:, cu[-1]:].any(), n


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,HV,gate_div,h0_std,forced', [
    (1, 2048, 2, 4, 2.0, 0.5, False),       # 16 workgroups of the scans: 4 segments of 8 chunks, automatic
    (2, 1100, 2, 2, 1.0, 0.5, True),        # ragged last chunk, segments of 4 chunks forced
    (1, 1024, 1, 2, 512.0, 0.5, True),      # hardly any decay: no segment may start warm, segment 0's workgroups walk the sequence
    (1, 1536, 2, 2, 16.0, None, True),      # slower decay: warm-ups of several chunks, the first and last reach the ends of the sequence
])
def test_chunk_backward_time_segments(B, T, H, HV, gate_div, h0_std, forced, monkeypatch):
    """The two scans cut into time segments that start from a zero state where the chunks' transition bounds allow it:
    against the oracle, and against the same call with whole sequences (equal up to what a warm start forgets, 2^-32)."""
    D = 128
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, D, D, seed=T, gate_div=gate_div, h0_std=h0_std)
    q, k, v = q.bfloat16(), k.bfloat16(), v.bfloat16()
    gen = torch.Generator().manual_seed(T + 1)
    do = torch.randn(B, T, HV, D, generator=gen).bfloat16()
    dht = torch.randn(B, HV, D, D, generator=gen)
    ref = O.gated_delta_rule_grads(q, k, v, g, beta, do, dht, initial_state=h0, dtype=torch.float32)
    got = {}
    for mode in ('segments' if forced else 'auto', 'wide'):
        monkeypatch.setenv('FLA_HIP_BWD_SCAN_MODE', mode)
        _, _, got[mode] = _grads_gpu(q, k, v, g, beta, h0, do, dht)
        _compare(ref, got[mode])
    a, b = got['segments' if forced else 'auto'], got['wide']
    for n in a:
        if a[n] is not None:
            assert O.get_err_ratio(b[n].float().cpu(), a[n].float().cpu()) < 2e-3, n

