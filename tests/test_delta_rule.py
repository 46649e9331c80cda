"""The delta rule without gates (chunk_delta_rule, fused_recurrent_delta_rule) on the gated operator's HIP
kernels, against the CPU oracle with g absent.  Shapes and input recipe of the reference's own matrix
(tests/ops/test_delta.py:15-95: fp16, normalised q and k, random initial state, bar 0.006)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O


def test_oracle_without_gate_is_the_plain_delta_rule():
    # closed form of fla/ops/delta_rule/naive.py:12-37: S += k (beta (v - S^T k))^T, o = S^T q scale
    torch.manual_seed(1)
    T, K, V = 6, 3, 2
    q, k = torch.randn(1, T, 1, K, dtype=torch.float64), F.normalize(torch.randn(1, T, 1, K, dtype=torch.float64), dim=-1)
    v, beta = torch.randn(1, T, 1, V, dtype=torch.float64), torch.rand(1, T, 1, dtype=torch.float64)
    S = torch.randn(K, V, dtype=torch.float64)
    o_ref, S_ref = torch.zeros(T, V, dtype=torch.float64), S.clone()
    for t in range(T):
        kt, qt = k[0, t, 0], q[0, t, 0]
        S_ref = S_ref + torch.outer(kt, beta[0, t, 0] * (v[0, t, 0] - S_ref.T @ kt))
        o_ref[t] = S_ref.T @ qt * K ** -0.5
    o, ht = O.recurrent_gated_delta_rule(q, k, v, None, beta, None, S[None, None], True, dtype=torch.float64)
    assert torch.allclose(o[0, :, 0], o_ref) and torch.allclose(ht[0, 0], S_ref)
    o0, ht0 = O.recurrent_gated_delta_rule(q, k, v, torch.zeros(1, T, 1), beta, None, S[None, None], True, dtype=torch.float64)
    assert torch.equal(o, o0) and torch.equal(ht, ht0)
    oc, hc = O.chunk_gated_delta_rule(q, k, v, torch.zeros(1, T, 1), beta, None, S[None, None], True, chunk_size=4, dtype=torch.float64)
    assert torch.allclose(oc, o) and torch.allclose(hc, ht)


def _check(name, ref, got, ratio):
    got = got.detach().float().cpu()
    assert not torch.isnan(got).any(), f'{name}: NaN'
    r, m = O.get_err_ratio(ref, got), O.max_abs_ratio(ref, got)
    assert r <= ratio and m <= 1e-2, f'{name}: rel-rmse {r:.3e} max-abs ratio {m:.3e}'


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,D,scale,l2,dtype', [
    (1, 63, 1, 64, 1, False, torch.float16),
    (2, 100, 4, 60, 0.1, False, torch.float16),
    (2, 1000, 3, 128, 0.1, False, torch.float16),
    (2, 1024, 4, 128, 1, True, torch.float16),
    (3, 2000, 4, 128, 0.1, False, torch.float16),
    (4, 2048, 8, 64, 0.1, False, torch.float16),
    (1, 700, 2, 128, 0.1, True, torch.bfloat16),
])
def test_chunk_delta_rule_reference_matrix(B, T, H, D, scale, l2, dtype):
    from fla_hip.ops.delta_rule import chunk_delta_rule, fused_recurrent_delta_rule
    gen = torch.Generator().manual_seed(42)
    q = torch.randn(B, T, H, D, generator=gen)
    k = torch.randn(B, T, H, D, generator=gen)
    v = torch.randn(B, T, H, D, generator=gen).to(dtype)
    beta = torch.randn(B, T, H, generator=gen).sigmoid().to(dtype)
    h0 = torch.randn(B, H, D, D, generator=gen)
    if not l2:
        q, k = F.normalize(q, dim=-1), F.normalize(k, dim=-1)
    q, k = q.to(dtype), k.to(dtype)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, None, beta, scale, h0, True, use_qk_l2norm_in_kernel=l2)
    dev = 'cuda'
    o, ht = chunk_delta_rule(q.to(dev), k.to(dev), v.to(dev), beta.to(dev), scale=scale, initial_state=h0.to(dev),
                             output_final_state=True, use_qk_l2norm_in_kernel=l2)
    assert o.dtype == dtype and ht.dtype == torch.float32
    _check('o', ref_o, o, 5e-3)
    _check('ht', ref_ht, ht, 5e-3)
    o2, ht2 = fused_recurrent_delta_rule(q.to(dev), k.to(dev), v.to(dev), beta.to(dev), scale=scale, initial_state=h0.to(dev),
                                         output_final_state=True, use_qk_l2norm_in_kernel=l2)
    _check('o recurrent', ref_o, o2, 2e-3)
    _check('ht recurrent', ref_ht, ht2, 2e-3)


@pytest.mark.gpu
def test_chunk_delta_rule_packed_and_validation():
    from fla_hip.ops.delta_rule import chunk_delta_rule
    dev = 'cuda'
    cu = [0, 100, 101, 400, 777]
    H, D = 2, 128
    gen = torch.Generator().manual_seed(3)
    q = F.normalize(torch.randn(1, cu[-1], H, D, generator=gen), dim=-1).bfloat16()
    k = F.normalize(torch.randn(1, cu[-1], H, D, generator=gen), dim=-1).bfloat16()
    v = torch.randn(1, cu[-1], H, D, generator=gen).bfloat16()
    beta = torch.rand(1, cu[-1], H, generator=gen)
    h0 = torch.randn(4, H, D, D, generator=gen)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, None, beta, None, h0, True, cu_seqlens=cu)
    for idx in (torch.int32, torch.int64):
        o, ht = chunk_delta_rule(q.to(dev), k.to(dev), v.to(dev), beta.to(dev), initial_state=h0.to(dev), output_final_state=True,
                                 cu_seqlens=torch.tensor(cu, dtype=idx, device=dev))
        _check('o', ref_o, o, 5e-3)
        _check('ht', ref_ht, ht, 5e-3)
    with pytest.raises(AssertionError):
        chunk_delta_rule(q.float().to(dev), k.float().to(dev), v.float().to(dev), beta.to(dev))
    with pytest.raises(ValueError):
        chunk_delta_rule(q.to(dev), k.to(dev), v.to(dev), beta.to(dev), chunk_size=48)
    with pytest.raises(ValueError):
        chunk_delta_rule(q.to(dev), k.to(dev), v.to(dev), beta.to(dev), initial_state=h0[:3].to(dev),
                         cu_seqlens=torch.tensor(cu, device=dev))


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,D,scale,l2,dtype', [
    (2, 100, 4, 60, 0.1, False, torch.float16),
    (2, 500, 3, 128, 0.1, False, torch.float16),
    (1, 300, 2, 128, 1, True, torch.bfloat16),
])
def test_chunk_delta_rule_backward(B, T, H, D, scale, l2, dtype):
    """Gradients through the operator against reverse-mode differentiation of the oracle's recurrence without a gate
    (the reference checks its backward the same way, bars 0.008: tests/ops/test_delta.py:60-86)."""
    from fla_hip.ops.delta_rule import chunk_delta_rule
    gen = torch.Generator().manual_seed(7)
    q, k = torch.randn(B, T, H, D, generator=gen), torch.randn(B, T, H, D, generator=gen)
    if not l2:
        q, k = F.normalize(q, dim=-1), F.normalize(k, dim=-1)
    q, k = q.to(dtype), k.to(dtype)
    v = torch.randn(B, T, H, D, generator=gen).to(dtype)
    beta = torch.rand(B, T, H, generator=gen).sigmoid()
    h0 = torch.randn(B, H, D, D, generator=gen) * 0.3
    do = torch.randn(B, T, H, D, generator=gen).to(dtype)
    dht = torch.randn(B, H, D, D, generator=gen)
    ref = O.gated_delta_rule_grads(q, k, v, None, beta, do, dht, scale=scale, initial_state=h0, use_qk_l2norm_in_kernel=l2,
                                   dtype=torch.float32)
    dev = 'cuda'
    leaves = [x.to(dev).requires_grad_(True) for x in (q, k, v, beta, h0)]
    o, ht = chunk_delta_rule(leaves[0], leaves[1], leaves[2], leaves[3], scale=scale, initial_state=leaves[4],
                             output_final_state=True, use_qk_l2norm_in_kernel=l2)
    ((o.float() * do.to(dev).float()).sum() + (ht * dht.to(dev)).sum()).backward()
    for name, x in zip(('dq', 'dk', 'dv', 'dbeta', 'dh0'), leaves):
        r = O.get_err_ratio(ref[name], x.grad.float().cpu())
        assert r <= 0.008, f'{name}: rel-rmse {r:.3e}'


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,K,V,scale,l2,dtype,what', [
    (1, 63, 1, 64, 64, 1, False, torch.float16, ''),
    (2, 100, 4, 60, 60, 0.1, False, torch.float16, ''),
    (2, 300, 3, 128, 128, 0.1, False, torch.float16, ''),
    (2, 256, 4, 128, 128, 1, True, torch.float16, ''),
    (2, 200, 2, 64, 128, 0.1, False, torch.float32, ''),
    (1, 150, 2, 256, 64, 0.1, True, torch.bfloat16, ''),
    (2, 130, 2, 100, 72, 0.1, False, torch.float32, 'beta_vector'),
    (2, 130, 2, 192, 40, 0.1, False, torch.float16, 'beta_vector'),
    (2, 90, 2, 64, 64, 0.1, False, torch.float32, 'no_beta'),
    (2, 90, 2, 64, 64, 0.1, True, torch.float32, 'no_h0'),
])
def test_fused_recurrent_delta_rule_backward(B, T, H, K, V, scale, l2, dtype, what):
    """Gradients through fused_recurrent_delta_rule (the kernel behind fla/ops/delta_rule/fused_recurrent.py:313-441, which
    the reference's own tests use as the truth for its chunked operator, tests/ops/test_delta.py:60-86) against
    reverse-mode differentiation of the oracle's recurrence without a gate.  The kernel computes in fp32 from the inputs
    as given, so the bar is far below the reference's 0.008."""
    from fla_hip.ops.delta_rule import fused_recurrent_delta_rule
    gen = torch.Generator().manual_seed(11)
    q, k = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen)
    if not l2:
        q, k = F.normalize(q, dim=-1), F.normalize(k, dim=-1)
    q, k = q.to(dtype), k.to(dtype)
    v = torch.randn(B, T, H, V, generator=gen).to(dtype)
    beta = torch.rand(B, T, H, V if what == 'beta_vector' else 1, generator=gen).sigmoid()
    beta = None if what == 'no_beta' else (beta if what == 'beta_vector' else beta[..., 0])
    h0 = None if what == 'no_h0' else torch.randn(B, H, K, V, generator=gen) * 0.3
    do = torch.randn(B, T, H, V, generator=gen).to(dtype)
    dht = torch.randn(B, H, K, V, generator=gen)
    ref = O.gated_delta_rule_grads(q, k, v, None, beta, do, dht, scale=scale, initial_state=h0, use_qk_l2norm_in_kernel=l2,
                                   dtype=torch.float64)
    dev = 'cuda'
    names = ('dq', 'dk', 'dv', 'dbeta', 'dh0')
    leaves = [None if x is None else x.to(dev).requires_grad_(True) for x in (q, k, v, beta, h0)]
    o, ht = fused_recurrent_delta_rule(leaves[0], leaves[1], leaves[2], leaves[3], scale=scale, initial_state=leaves[4],
                                       output_final_state=True, use_qk_l2norm_in_kernel=l2)
    ((o.float() * do.to(dev).float()).sum() + (ht * dht.to(dev)).sum()).backward()
    for name, x in zip(names, leaves):
        if x is None:
            continue
        assert x.grad.shape == x.shape and x.grad.dtype == x.dtype
        got = x.grad.double().cpu()
        assert not torch.isnan(got).any(), name
        r = O.get_err_ratio(ref[name], got)
        # (16-bit gradients carry their own rounding: 2^-9 relative for bf16)
        bar = 2e-5 if dtype == torch.float32 else 3e-3 if dtype == torch.bfloat16 and name in ('dq', 'dk', 'dv') else 1e-3
        assert r <= bar, f'{name}: rel-rmse {r:.3e} > {bar}'


@pytest.mark.gpu
def test_fused_recurrent_delta_rule_backward_packed():
    # packed sequences with tokens in front of the first and behind the last one (zero gradients there), an empty and a
    # one-token sequence; every sequence's gradients are those of the sequence alone
    from fla_hip.ops.delta_rule import fused_recurrent_delta_rule
    cu, T, H, D = [30, 30, 31, 200, 333], 350, 2, 64
    N = len(cu) - 1
    gen = torch.Generator().manual_seed(12)
    q = F.normalize(torch.randn(1, T, H, D, generator=gen), dim=-1)
    k = F.normalize(torch.randn(1, T, H, D, generator=gen), dim=-1)
    v = torch.randn(1, T, H, D, generator=gen)
    beta = torch.rand(1, T, H, generator=gen).sigmoid()
    h0 = torch.randn(N, H, D, D, generator=gen) * 0.3
    do, dht = torch.randn(1, T, H, D, generator=gen), torch.randn(N, H, D, D, generator=gen)
    sl = slice(cu[0], cu[-1])
    ref = O.gated_delta_rule_grads(q[:, sl], k[:, sl], v[:, sl], None, beta[:, sl], do[:, sl], dht, initial_state=h0,
                                   cu_seqlens=[c - cu[0] for c in cu], dtype=torch.float64)
    dev = 'cuda'
    for idx in (torch.int32, torch.int64):
        junk = [torch.full((1, T, H, D), float('nan'), device=dev) for _ in range(6)]       # what an uninitialised buffer would show
        del junk
        leaves = [x.to(dev).requires_grad_(True) for x in (q, k, v, beta, h0)]
        o, ht = fused_recurrent_delta_rule(*leaves[:4], initial_state=leaves[4], output_final_state=True,
                                           cu_seqlens=torch.tensor(cu, dtype=idx, device=dev))
        ((o[:, sl] * do[:, sl].to(dev)).sum() + (ht * dht.to(dev)).sum()).backward()
        for name, x in zip(('dq', 'dk', 'dv', 'dbeta'), leaves):
            got = x.grad.double().cpu()
            assert not torch.isnan(got).any(), name
            assert not got[:, :cu[0]].any() and not got[:, cu[-1]:].any(), f'{name}: tokens outside the sequences'
            r = O.get_err_ratio(ref[name], got[:, sl])
            assert r <= 2e-5, f'{name}: rel-rmse {r:.3e}'
        assert O.get_err_ratio(ref['dh0'], leaves[4].grad.double().cpu()) <= 2e-5
        assert torch.equal(leaves[4].grad[0].cpu(), dht[0])          # the empty sequence hands its state gradient through
