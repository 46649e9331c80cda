"""GPU parity of fused_recurrent_gated_delta_rule (HIP, through the C ABI) against the CPU
oracle on the same seeded inputs.  Shapes follow the reference's own matrix
(tests/ops/test_gdn.py:48-105, :450-517) plus the decode configuration."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu

# tolerance on o and on the final state: relative RMSE <= 2e-3 (the reference's own bar for
# this kernel, tests/ops/test_gdn.py:104-105) and max-abs-error ratio <= 1e-2
RATIO, MAXABS = 2e-3, 1e-2


def _ops():
    from fla_hip.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    return fused_recurrent_gated_delta_rule


def _check(name, ref, got, ratio=RATIO):
    got = got.detach().float().cpu()
    assert not torch.isnan(got).any(), f'{name}: NaN'
    r, m = O.get_err_ratio(ref, got), O.max_abs_ratio(ref, got)
    assert r <= ratio and m <= MAXABS, f'{name}: rel-rmse {r:.3e} max-abs ratio {m:.3e}'


def _inputs(B, T, H, HV, D, dtype, seed=42, gate_norm=1.0):
    gen = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, D, generator=gen).to(dtype)
    k = torch.randn(B, T, H, D, generator=gen).to(dtype)
    v = torch.randn(B, T, HV, D, generator=gen).to(dtype)
    beta = torch.rand(B, T, HV, generator=gen).sigmoid()
    g = F.logsigmoid(torch.rand(B, T, HV, generator=gen)) / gate_norm
    h0 = torch.randn(B, HV, D, D, generator=gen)
    return q, k, v, g, beta, h0


@pytest.mark.parametrize('B,T,H,HV,D,scale,gate_norm,dtype', [
    (1, 63, 1, 1, 64, 1.0, 1.0, torch.float32),
    (2, 200, 4, 4, 60, 1.0, 1.0, torch.float32),
    (2, 300, 2, 8, 128, 1.0, 0.1, torch.float32),
    (3, 256, 2, 2, 128, 0.1, 1.0, torch.float32),
    (2, 128, 3, 3, 100, 1.0, 10.0, torch.float32),
    (2, 256, 4, 4, 128, 0.1, 1.0, torch.float16),
    (2, 256, 4, 8, 128, 1.0, 10.0, torch.float16),
    (2, 256, 2, 4, 128, 1.0, 1.0, torch.bfloat16),
    (1, 64, 2, 2, 256, 1.0, 1.0, torch.float32),
])
def test_fused_recurrent_vs_oracle(B, T, H, HV, D, scale, gate_norm, dtype):
    op = _ops()
    q, k, v, g, beta, h0 = _inputs(B, T, H, HV, D, dtype, gate_norm=gate_norm)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, scale, h0, True, use_qk_l2norm_in_kernel=True)
    dev = 'cuda'
    o, ht = op(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), scale=scale,
               initial_state=h0.to(dev), output_final_state=True, use_qk_l2norm_in_kernel=True)
    assert o.dtype == v.dtype and ht.dtype == torch.float32 and ht.shape == (B, HV, D, D)
    ratio = RATIO if dtype == torch.float32 else 5e-3      # o itself is rounded to 16 bits
    _check('o', ref_o, o, ratio)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('B,T,H,HV,D,scale,gate_logit_normalizer,dtype', [
    (1, 63, 1, 1, 64, 1, 1, torch.float),
    (2, 500, 4, 4, 60, 1, 1, torch.float),
    (2, 1000, 2, 8, 128, 1, 0.1, torch.float),
    (3, 1024, 2, 2, 128, 0.1, 1, torch.float),
    (4, 1024, 3, 3, 128, 1, 10, torch.float),
    (4, 2048, 4, 4, 64, 0.1, 1, torch.float),
    (2, 1024, 4, 4, 128, 1, 0.1, torch.float16),
    (2, 1024, 4, 8, 128, 1, 10, torch.float16),
])
def test_reference_matrix_with_the_reference_input_recipe(B, T, H, HV, D, scale, gate_logit_normalizer, dtype):
    """The reference's own matrix and recipe for this operator (tests/ops/test_gdn.py:48-105): q and k in
    fp32 and NOT normalised (the kernel does it), v and beta in the test dtype, unit-variance fp32 initial
    state, full sequence lengths.  Its bar: error ratio 0.002 on o and ht."""
    gen = torch.Generator().manual_seed(42)
    q = torch.randn(B, T, H, D, generator=gen)
    k = torch.randn(B, T, H, D, generator=gen)
    v = torch.randn(B, T, HV, D, generator=gen).to(dtype)
    beta = torch.rand(B, T, HV, generator=gen).to(dtype).sigmoid()
    g = F.logsigmoid(torch.rand(B, T, HV, generator=gen)) / gate_logit_normalizer
    h0 = torch.randn(B, HV, D, D, generator=gen)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(F.normalize(q, p=2, dim=-1).to(dtype), F.normalize(k, p=2, dim=-1).to(dtype),
                                                 v, g, beta, scale, h0, True)
    dev = 'cuda'
    o, ht = _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), scale=scale,
                   initial_state=h0.to(dev), output_final_state=True, use_qk_l2norm_in_kernel=True)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('B,T,H,HV,D,scale,has_dt_bias,neg_eigval,dtype', [
    (1, 64, 1, 1, 64, 1, False, False, torch.float),
    (2, 256, 2, 2, 64, 1, True, False, torch.float),
    (2, 512, 2, 4, 64, 0.1, True, True, torch.float16),
    (3, 1000, 2, 8, 128, 1, False, True, torch.float16),
    (4, 1024, 4, 4, 128, 0.1, True, False, torch.float16),
])
def test_reference_in_kernel_gate_and_beta_matrices(B, T, H, HV, D, scale, has_dt_bias, neg_eigval, dtype):
    """tests/ops/test_gdn.py:520-657: raw gates with A_log = log U(1, 16) and optional dt_bias activated in
    the kernel, and beta logits squashed in the kernel (doubled with allow_neg_eigval), both on top of
    the in-kernel l2 normalisation, against the oracle fed with the activated values.  Bar 0.002."""
    gen = torch.Generator().manual_seed(42)
    q = torch.randn(B, T, H, D, generator=gen).to(dtype)
    k = torch.randn(B, T, H, D, generator=gen).to(dtype)
    v = torch.randn(B, T, HV, D, generator=gen).to(dtype)
    beta_logits = torch.randn(B, T, HV, generator=gen).to(dtype)
    g_raw = torch.randn(B, T, HV, generator=gen)
    A_log = torch.log(torch.empty(HV).uniform_(1, 16, generator=gen))
    dt_bias = torch.randn(HV, generator=gen) if has_dt_bias else None
    h0 = torch.randn(B, HV, D, D, generator=gen)
    g_ref = -A_log.exp() * F.softplus(g_raw + (dt_bias if has_dt_bias else 0.0))
    beta_ref = beta_logits.float().sigmoid() * (2.0 if neg_eigval else 1.0)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g_ref, beta_ref, scale, h0, True, use_qk_l2norm_in_kernel=True)
    dev = 'cuda'
    o, ht = _ops()(q.to(dev), k.to(dev), v.to(dev), g_raw.to(dev), beta=beta_logits.to(dev), scale=scale,
                   initial_state=h0.to(dev), output_final_state=True, use_qk_l2norm_in_kernel=True,
                   use_gate_in_kernel=True, A_log=A_log.to(dev), dt_bias=None if dt_bias is None else dt_bias.to(dev),
                   use_beta_sigmoid_in_kernel=True, allow_neg_eigval=neg_eigval)
    ratio = RATIO if dtype == torch.float32 else 5e-3      # o itself is rounded to 16 bits
    _check('o', ref_o, o, ratio)
    _check('ht', ref_ht, ht)


def test_decode_shape_inplace_and_chained_steps():
    """N=64 decode steps with Hqk=16, Hv=32, K=V=128 (the decode configuration at a quarter
    of its batch): three chained single-token calls, state updated in place, must equal the
    oracle's three-token recurrence."""
    op = _ops()
    N, H, HV, D = 64, 16, 32, 128
    gen = torch.Generator().manual_seed(1)
    q = F.normalize(torch.randn(N, 3, H, D, generator=gen), dim=-1).bfloat16()
    k = F.normalize(torch.randn(N, 3, H, D, generator=gen), dim=-1).bfloat16()
    v = torch.randn(N, 3, HV, D, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(N, 3, HV, generator=gen))
    beta = torch.sigmoid(torch.randn(N, 3, HV, generator=gen))
    h0 = 0.1 * torch.randn(N, HV, D, D, generator=gen)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    dev = 'cuda'
    state = h0.to(dev)
    ptr0 = state.data_ptr()
    outs = []
    for t in range(3):
        o, st = op(q[:, t:t + 1].to(dev), k[:, t:t + 1].to(dev), v[:, t:t + 1].to(dev), g[:, t:t + 1].to(dev),
                   beta=beta[:, t:t + 1].to(dev), initial_state=state, output_final_state=True, inplace_final_state=True)
        assert st.data_ptr() == ptr0
        outs.append(o)
    _check('o', ref_o, torch.cat(outs, 1), 5e-3)
    _check('ht', ref_ht, state)
    # one 3-token call gives the same state as the three chained calls, bit for bit
    o3, st3 = op(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), initial_state=h0.to(dev),
                 output_final_state=True)
    assert torch.equal(st3, state) and torch.equal(o3, torch.cat(outs, 1))


@pytest.mark.parametrize('cu,H,HV,D', [
    ([0, 15], 2, 2, 64),
    ([0, 1, 100, 101, 300], 2, 4, 64),
    ([0, 15, 100, 300, 1200, 1500], 2, 8, 100),
])
@pytest.mark.parametrize('idx_dtype', [torch.int64, torch.int32])
def test_varlen_ownership_is_bit_exact(cu, H, HV, D, idx_dtype):
    """Packed call == each sequence run alone, bit for bit, and both match the oracle."""
    op = _ops()
    T, N = cu[-1], len(cu) - 1
    q, k, v, g, beta, _ = _inputs(1, T, H, HV, D, torch.float16, seed=3)
    h0 = torch.randn(N, HV, D, D, generator=torch.Generator().manual_seed(4))
    dev = 'cuda'
    a = [x.to(dev) for x in (q, k, v, g, beta)]
    o, ht = op(a[0], a[1], a[2], a[3], beta=a[4], initial_state=h0.to(dev), output_final_state=True,
               use_qk_l2norm_in_kernel=True, cu_seqlens=torch.tensor(cu, dtype=idx_dtype, device=dev))
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu_seqlens=cu,
                                                 use_qk_l2norm_in_kernel=True)
    _check('o', ref_o, o, 5e-3)
    _check('ht', ref_ht, ht)
    for n, (s, e) in enumerate(zip(cu[:-1], cu[1:])):
        o_n, h_n = op(a[0][:, s:e], a[1][:, s:e], a[2][:, s:e], a[3][:, s:e], beta=a[4][:, s:e],
                      initial_state=h0[n:n + 1].to(dev), output_final_state=True, use_qk_l2norm_in_kernel=True)
        assert torch.equal(o_n[0], o[0, s:e]), f'sequence {n}: o differs'
        assert torch.equal(h_n[0], ht[n]), f'sequence {n}: state differs'


def test_flags_gate_sigmoid_vector_beta_gk_gv_vfirst():
    op = _ops()
    B, T, H, HV, D = 2, 70, 2, 4, 64
    gen = torch.Generator().manual_seed(5)
    q, k = torch.randn(B, T, H, D, generator=gen), torch.randn(B, T, H, D, generator=gen)
    v = torch.randn(B, T, HV, D, generator=gen)
    graw, braw = torch.randn(B, T, HV, generator=gen), torch.randn(B, T, HV, D, generator=gen)
    gk = -0.1 * torch.rand(B, T, HV, D, generator=gen)
    gv = -0.1 * torch.rand(B, T, HV, D, generator=gen)
    A_log, dt_bias = 0.3 * torch.randn(HV, generator=gen), 0.3 * torch.randn(HV, generator=gen)
    h0 = torch.randn(B, HV, D, D, generator=gen)
    kw = dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True, A_log=A_log, dt_bias=dt_bias,
              use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, graw, braw, None, h0, True, gk=gk, gv=gv, **kw)
    dev = 'cuda'
    kwd = dict(kw, A_log=A_log.to(dev), dt_bias=dt_bias.to(dev))
    o, ht = op(q.to(dev), k.to(dev), v.to(dev), graw.to(dev), gk=gk.to(dev), gv=gv.to(dev), beta=braw.to(dev),
               initial_state=h0.to(dev), output_final_state=True, **kwd)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    # V-first layout is the transpose of the default one
    o2, ht2 = op(q.to(dev), k.to(dev), v.to(dev), graw.to(dev), gk=gk.to(dev), gv=gv.to(dev), beta=braw.to(dev),
                 initial_state=h0.transpose(-1, -2).contiguous().to(dev), output_final_state=True,
                 state_v_first=True, **kwd)
    _check('o (v-first)', ref_o, o2)
    _check('ht (v-first)', ref_ht.transpose(-1, -2), ht2)
    # no gate, no beta: plain delta rule with beta = 1
    ref_o, ref_ht = O.recurrent_gated_delta_rule(O.l2norm(q), O.l2norm(k), v, None, None, None, None, True)
    o, ht = op(O.l2norm(q).to(dev), O.l2norm(k).to(dev), v.to(dev), output_final_state=True)
    _check('o (no g/beta)', ref_o, o)
    _check('ht (no g/beta)', ref_ht, ht)
    o, none = op(q.to(dev), k.to(dev), v.to(dev), graw.to(dev) * 0 - 0.1)
    assert none is None


@pytest.mark.parametrize('idx_dtype', [torch.int32, torch.int64])
@pytest.mark.parametrize('vfirst,cu', [(False, None), (True, None), (False, [0, 3, 4, 9])])
def test_state_pool_addressed_by_slot(idx_dtype, vfirst, cu):
    """Continuous batching: every sequence names its slot in a state pool; the step reads and writes
    that slot in place and touches no other (fla/ops/kda/fused_recurrent.py:75-91,145-159 for the
    sibling operator; the GDN reference has no such argument)."""
    H, HV, D, slots_total = 2, 4, 128, 11
    N = 3
    if cu is None:
        q, k, v, g, beta, _ = _inputs(N, 2, H, HV, D, torch.bfloat16, seed=9)
    else:
        q, k, v, g, beta, _ = _inputs(1, cu[-1], H, HV, D, torch.bfloat16, seed=9)
    gen = torch.Generator().manual_seed(10)
    pool = torch.randn(slots_total, HV, D, D, generator=gen)
    slots = [7, 0, 4]
    ref_o, ref_h = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, pool[slots], True, cu_seqlens=cu)
    dev = 'cuda'
    dpool = (pool.transpose(-1, -2) if vfirst else pool).contiguous().to(dev)
    before = dpool.clone()
    o, out = _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), initial_state=dpool,
                    output_final_state=True, inplace_final_state=True, state_v_first=vfirst,
                    cu_seqlens=None if cu is None else torch.tensor(cu, device=dev),
                    ssm_state_indices=torch.tensor(slots, dtype=idx_dtype, device=dev))
    assert out.data_ptr() == dpool.data_ptr()
    _check('o', ref_o, o)
    got = dpool[slots].transpose(-1, -2) if vfirst else dpool[slots]
    _check('slots', ref_h, got)
    rest = [i for i in range(slots_total) if i not in slots]
    assert torch.equal(dpool[rest], before[rest]), 'a slot that no sequence named was modified'
    with pytest.raises(ValueError):
        _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), initial_state=dpool,
               output_final_state=True, ssm_state_indices=torch.tensor(slots, device=dev))


@pytest.mark.parametrize('idx_dtype', [torch.int32, torch.int64])
@pytest.mark.parametrize('vfirst,cu', [(False, None), (True, None), (False, [0, 3, 4, 6])])
def test_speculative_decoding_slot_per_token(idx_dtype, vfirst, cu):
    """ssm_state_indices [N, T] with num_accepted_tokens (fla/ops/kda/fused_recurrent.py:131-145,203-219):
    each sequence starts from the slot of its last accepted token and leaves the state after draft
    token t in slot [n, t]; slots nobody writes keep their contents."""
    H, HV, D, slots_total, N, TMAX = 2, 4, 128, 16, 3, 3
    gen = torch.Generator().manual_seed(21)
    pool = torch.randn(slots_total, HV, D, D, generator=gen)
    idx = torch.randperm(slots_total, generator=gen)[:N * TMAX].view(N, TMAX)
    accepted = torch.tensor([2, 1, 3])
    if cu is None:
        q, k, v, g, beta, _ = _inputs(N, TMAX, H, HV, D, torch.bfloat16, seed=11)
        lens = [TMAX] * N
    else:
        q, k, v, g, beta, _ = _inputs(1, cu[-1], H, HV, D, torch.bfloat16, seed=11)
        lens = [b - a for a, b in zip(cu[:-1], cu[1:])]
        accepted = torch.tensor([2, 1, 2])
    ref_o, ref_pool, ref_tok = O.recurrent_gated_delta_rule_pooled(q, k, v, g, beta, None, pool, idx, accepted, cu_seqlens=cu)
    dev = 'cuda'
    lay = (lambda x: x.transpose(-1, -2).contiguous()) if vfirst else (lambda x: x.contiguous())
    dpool = lay(pool).to(dev)
    before = dpool.clone()
    kw = dict(beta=beta.to(dev), state_v_first=vfirst, cu_seqlens=None if cu is None else torch.tensor(cu, device=dev),
              ssm_state_indices=idx.to(device=dev, dtype=idx_dtype), num_accepted_tokens=accepted.to(dev))
    # read-only pool: a state per token comes back
    o, per_tok = _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), initial_state=dpool, **kw)
    assert torch.equal(dpool, before)
    _check('o', ref_o, o)
    _check('per-token states', lay(ref_tok), per_tok)
    # in place: slot [n, t] receives the state after token t
    o2, out = _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), initial_state=dpool, inplace_final_state=True, **kw)
    assert out.data_ptr() == dpool.data_ptr() and torch.equal(o2, o)
    written = sorted({int(idx[n, t]) for n in range(N) for t in range(lens[n])})
    rest = [i for i in range(slots_total) if i not in written]
    _check('pool', lay(ref_pool)[written], dpool[written])
    assert torch.equal(dpool[rest], before[rest]), 'a slot that no token named was modified'
    with pytest.raises(ValueError):
        _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), initial_state=dpool, beta=beta.to(dev),
               ssm_state_indices=idx[:, 0].to(dev), num_accepted_tokens=accepted.to(dev), inplace_final_state=True)


def test_spec_pool_scalar_fixture_on_the_gpu():
    import os
    import numpy as np
    gold = np.load(os.path.join(os.path.dirname(__file__), 'golden', 'gdn_scalar_cases_ext.npz'))
    t = lambda key: torch.from_numpy(gold[f'spec_pool.{key}'])
    dev = 'cuda'
    # the fixture has K = 2, V = 3; pooled states are updated in place, so the zero padding to multiples of 4
    # (which changes nothing else) is done here instead of inside the operator
    K, V = t('k').shape[-1], t('v').shape[-1]
    padk = lambda x: F.pad(x.float(), (0, 4 - K))
    pool = F.pad(t('pool').float(), (0, 4 - V, 0, 4 - K)).to(dev)
    o, _ = _ops()(padk(t('q'))[None].to(dev), padk(t('k'))[None].to(dev), F.pad(t('v').float(), (0, 4 - V))[None].to(dev),
                  t('g')[None].float().to(dev), beta=t('beta')[None].float().to(dev), scale=float(gold['spec_pool.scale']),
                  initial_state=pool, inplace_final_state=True, cu_seqlens=t('cu').to(dev),
                  ssm_state_indices=t('idx').to(dev), num_accepted_tokens=t('accepted').to(dev))
    _check('o', t('o')[None].float(), o[..., :V], 1e-5)
    _check('pool', t('pool_after').float(), pool[..., :K, :V], 1e-5)
    assert not pool[..., K:, :].any() and not pool[..., :, V:].any()


@pytest.mark.parametrize('name', ['gk_gv_vbeta', 'gk_only_varlen', 'gv_vbeta_varlen'])
@pytest.mark.parametrize('vfirst', [False, True])
def test_optional_decay_scalar_fixtures_on_the_gpu(name, vfirst):
    """gk, gv and beta per value column against the scalar fixtures directly (K and V are 2 or 3 there:
    the host pads head dims that are not multiples of 4)."""
    import os
    import numpy as np
    gold = np.load(os.path.join(os.path.dirname(__file__), 'golden', 'gdn_scalar_cases_ext.npz'))
    dev = 'cuda'
    t = lambda key: torch.from_numpy(gold[f'{name}.{key}'])[None].float().to(dev) if f'{name}.{key}' in gold.files else None
    h0 = torch.from_numpy(gold[f'{name}.h0']).float()
    o, ht = _ops()(t('q'), t('k'), t('v'), t('g'), gk=t('gk'), gv=t('gv'), beta=t('beta'), scale=float(gold[f'{name}.scale']),
                   initial_state=(h0.transpose(-1, -2).contiguous() if vfirst else h0).to(dev), output_final_state=True,
                   state_v_first=vfirst, cu_seqlens=torch.from_numpy(gold[f'{name}.cu']).to(dev))
    _check('o', torch.from_numpy(gold[f'{name}.o'])[None].float(), o, 1e-5)
    ref_ht = torch.from_numpy(gold[f'{name}.ht']).float()
    _check('ht', ref_ht.transpose(-1, -2) if vfirst else ref_ht, ht, 1e-5)


@pytest.mark.parametrize('K,V', [(50, 30), (6, 130), (129, 3)])
def test_head_dims_that_are_not_multiples_of_four(K, V):
    # the reference takes any K <= 256 (BK = next_power_of_2(K), fla/ops/gated_delta_rule/fused_recurrent.py:206-208)
    gen = torch.Generator().manual_seed(K * 1000 + V)
    B, T, H, HV = 2, 5, 1, 2
    q, k = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen)
    v = torch.randn(B, T, HV, V, generator=gen)
    g, beta = -torch.rand(B, T, HV, generator=gen), torch.rand(B, T, HV, generator=gen)
    h0 = torch.randn(B, HV, K, V, generator=gen)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, use_qk_l2norm_in_kernel=True)
    dev = 'cuda'
    o, ht = _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), initial_state=h0.to(dev),
                   output_final_state=True, use_qk_l2norm_in_kernel=True)
    assert o.shape == ref_o.shape and ht.shape == ref_ht.shape
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('vfirst', [False, True])
def test_missing_beta_counts_as_ones_before_the_sigmoid(vfirst):
    # fla/ops/gated_delta_rule/fused_recurrent.py:443: beta = ones, then the in-kernel sigmoid still applies
    q, k, v, g, _, h0 = _inputs(2, 3, 2, 4, 64, torch.float32, seed=3)
    dev = 'cuda'
    for neg in (False, True):
        ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, torch.ones(2, 3, 4), None, h0, True,
                                                     use_beta_sigmoid_in_kernel=True, allow_neg_eigval=neg,
                                                     use_qk_l2norm_in_kernel=True)
        st = h0.transpose(-1, -2).contiguous() if vfirst else h0
        o, ht = _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), initial_state=st.to(dev), output_final_state=True,
                       use_beta_sigmoid_in_kernel=True, allow_neg_eigval=neg, use_qk_l2norm_in_kernel=True, state_v_first=vfirst)
        _check('o', ref_o, o)
        _check('ht', ref_ht.transpose(-1, -2) if vfirst else ref_ht, ht)


def test_no_tokens_returns_the_initial_state():
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    dev = 'cuda'
    h0 = torch.randn(2, 4, 64, 64, device=dev)
    e = lambda *shape: torch.empty(*shape, device=dev, dtype=torch.bfloat16)
    for op in (_ops(), chunk_gated_delta_rule):
        poison = torch.full((1 << 20,), float('nan'), device=dev); del poison       # what torch.empty may hand back
        o, ht = op(e(2, 0, 2, 64), e(2, 0, 2, 64), e(2, 0, 4, 64), e(2, 0, 4).float(), beta=e(2, 0, 4).float(),
                   initial_state=h0, output_final_state=True)
        assert o.shape == (2, 0, 4, 64) and torch.equal(ht, h0) and ht.data_ptr() != h0.data_ptr()
        o, ht = op(e(2, 0, 2, 64), e(2, 0, 2, 64), e(2, 0, 4, 64), e(2, 0, 4).float(), beta=e(2, 0, 4).float(),
                   output_final_state=True)
        assert torch.equal(ht, torch.zeros_like(h0))
    # packed input whose sequences are all empty
    cu = torch.zeros(3, dtype=torch.long, device=dev)
    o, ht = chunk_gated_delta_rule(e(1, 0, 2, 64), e(1, 0, 2, 64), e(1, 0, 4, 64), e(1, 0, 4).float(), e(1, 0, 4).float(),
                                   initial_state=h0, output_final_state=True, cu_seqlens=cu)
    assert torch.equal(ht, h0)


@pytest.mark.parametrize('vfirst', [False, True])
@pytest.mark.parametrize('case', ['plain', 'flags', 'packed', 'slots', 'f16', 'fp32'])
def test_decode_kernel_for_the_common_shape(case, vfirst):
    """K = V = 128, 1024 or more (sequence, head) states: the decode kernels written for that shape, one per state layout."""
    H, HV, D = 8, 32, 128
    dtype = {'f16': torch.float16, 'fp32': torch.float32}.get(case, torch.bfloat16)
    kw, okw = {}, {}
    cu = None
    if case == 'packed':
        lens = [1, 3, 2, 1] * 8
        cu = [0]
        for x in lens:
            cu.append(cu[-1] + x)
        q, k, v, g, beta, _ = _inputs(1, cu[-1], H, HV, D, dtype, seed=17)
        N = len(lens)
    else:
        N, T = 32, 2 if case != 'slots' else 1
        q, k, v, g, beta, _ = _inputs(N, T, H, HV, D, dtype, seed=17)
    gen = torch.Generator().manual_seed(18)
    h0 = torch.randn(N, HV, D, D, generator=gen)
    if case == 'flags':
        A_log, dt_bias = 0.3 * torch.randn(HV, generator=gen), 0.3 * torch.randn(HV, generator=gen)
        g, beta = torch.randn(g.shape, generator=gen), torch.randn(beta.shape, generator=gen)
        okw = dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True, A_log=A_log, dt_bias=dt_bias,
                   use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True)
        kw = dict(okw, A_log=A_log.cuda(), dt_bias=dt_bias.cuda())
    else:
        okw = kw = dict(use_qk_l2norm_in_kernel=True)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu_seqlens=cu, **okw)
    dev = 'cuda'
    cu_t = None if cu is None else torch.tensor(cu, device=dev)
    lay = (lambda x: x.transpose(-1, -2).contiguous()) if vfirst else (lambda x: x)
    kw = dict(kw, state_v_first=vfirst)
    if case == 'slots':
        pool = torch.randn(N + 5, HV, D, D, generator=gen)
        idx = torch.randperm(N + 5, generator=gen)[:N]
        pool[idx] = h0
        dpool = lay(pool).to(dev)
        o, _ = _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), initial_state=dpool, inplace_final_state=True,
                      ssm_state_indices=idx.to(dev), **kw)
        ht = dpool[idx.to(dev)]
        rest = [i for i in range(N + 5) if i not in idx.tolist()]
        assert torch.equal(dpool[rest].cpu(), lay(pool[rest]))
    else:
        o, ht = _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), initial_state=lay(h0).to(dev),
                       output_final_state=True, cu_seqlens=cu_t, **kw)
    _check('o', ref_o, o)
    _check('ht', ref_ht, lay(ht))


@pytest.mark.parametrize('case', ['plain', 'few', 'flags', 'packed', 'slots', 'f16'])
def test_decode_with_states_kept_in_bf16(case):
    """A bf16 state updated in place (an option of this library; the reference's GDN states are fp32): the step runs in
    fp32 from the bf16 values and the state is rounded once on the way back.  Checked against the fp32 oracle started
    from the same bf16 values: o to the usual bound, the state against the oracle's state rounded to bf16 (at most one
    unit in the last place apart wherever the fp32 results agree that closely), and over two calls in a row against
    the oracle with the rounding in between."""
    H, HV, D = 8, 32, 128
    dtype = torch.float16 if case == 'f16' else torch.bfloat16
    kw, okw = {}, {}
    cu = None
    N = 3 if case == 'few' else 67                       # 67 x 32 states: placed on the XCDs, the grid rounded up
    if case == 'packed':
        lens = [1, 3, 2, 1] * 8
        cu = [0]
        for x in lens:
            cu.append(cu[-1] + x)
        q, k, v, g, beta, _ = _inputs(1, cu[-1], H, HV, D, dtype, seed=27)
        N = len(lens)
    else:
        q, k, v, g, beta, _ = _inputs(N, 2, H, HV, D, dtype, seed=27)
    gen = torch.Generator().manual_seed(28)
    h0 = torch.randn(N, HV, D, D, generator=gen).bfloat16()
    if case == 'flags':
        A_log, dt_bias = 0.3 * torch.randn(HV, generator=gen), 0.3 * torch.randn(HV, generator=gen)
        g, beta = torch.randn(g.shape, generator=gen), torch.randn(beta.shape, generator=gen)
        okw = dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True, A_log=A_log, dt_bias=dt_bias,
                   use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True)
        kw = dict(okw, A_log=A_log.cuda(), dt_bias=dt_bias.cuda())
    else:
        okw = kw = dict(use_qk_l2norm_in_kernel=True)
    dev = 'cuda'
    cu_t = None if cu is None else torch.tensor(cu, device=dev)
    dq, dk, dv, dg, db = (x.to(dev) for x in (q, k, v, g, beta))

    def run(state, sl=slice(None)):
        if case == 'slots':
            pool = torch.randn(N + 5, HV, D, D, generator=gen).bfloat16()
            idx = torch.randperm(N + 5, generator=gen)[:N]
            pool[idx] = state
            dpool = pool.to(dev)
            o, ret = _ops()(dq[:, sl], dk[:, sl], dv[:, sl], dg[:, sl], beta=db[:, sl], initial_state=dpool,
                            inplace_final_state=True, ssm_state_indices=idx.to(dev), **kw)
            rest = [i for i in range(N + 5) if i not in idx.tolist()]
            assert torch.equal(dpool[rest].cpu(), pool[rest]), 'slots that are not named must keep their contents'
            return o, dpool[idx.to(dev)]
        dstate = state.to(dev)
        o, ret = _ops()(dq[:, sl], dk[:, sl], dv[:, sl], dg[:, sl], beta=db[:, sl], initial_state=dstate,
                        inplace_final_state=True, cu_seqlens=cu_t, **kw)
        assert ret.data_ptr() == dstate.data_ptr() and ret.dtype == torch.bfloat16
        return o, dstate

    def check_state(name, ref, got):
        got = got.cpu()
        assert got.dtype == torch.bfloat16 and not torch.isnan(got.float()).any()
        want = ref.bfloat16()
        # one unit in the last place of a bf16 value x is at most 2^-7 |x|
        off = (got.float() - want.float()).abs() > 2.0 ** -7 * want.float().abs() + 1e-6
        assert off.float().mean() < 1e-4, f'{name}: {int(off.sum())} of {off.numel()} elements more than one ulp off'
        assert (got == want).float().mean() > 0.98, f'{name}: only {(got == want).float().mean():.4f} rounded alike'
        assert O.get_err_ratio(ref, got.float()) <= 3e-3, name

    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0.float(), True, cu_seqlens=cu, **okw)
    o, ht = run(h0)
    _check('o', ref_o, o)
    check_state('ht', ref_ht, ht)
    if cu is None:
        # two calls of one token each: the state passes through bf16 in between
        r1_o, r1_h = O.recurrent_gated_delta_rule(q[:, :1], k[:, :1], v[:, :1], g[:, :1], beta[:, :1], None, h0.float(), True, **okw)
        o1, h1 = run(h0, slice(0, 1))
        check_state('ht after the first call', r1_h, h1)
        r2_o, r2_h = O.recurrent_gated_delta_rule(q[:, 1:], k[:, 1:], v[:, 1:], g[:, 1:], beta[:, 1:], None,
                                                  h1.cpu().float(), True, **okw)
        o2, h2 = run(h1.cpu(), slice(1, 2))
        _check('o of the second call', r2_o, o2)
        check_state('ht after the second call', r2_h, h2)


def test_bf16_states_are_refused_where_no_kernel_covers_them():
    dev = 'cuda'
    q, k, v, g, beta, _ = _inputs(2, 1, 2, 4, 64, torch.bfloat16, seed=1)
    h0 = torch.zeros(2, 4, 64, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(NotImplementedError, match='bf16 states need'):
        _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), initial_state=h0, inplace_final_state=True)
    # (straight through the C ABI as well)
    from fla_hip import _lib
    lib = _lib.load()
    rc = lib.gdn_fused_recurrent_fwd(*([None] * 9), h0.data_ptr(), h0.data_ptr(), None, None, None, None, 1,
                                     2, 0, 2, 4, 64, 64, 2, 1.0, 0, 0, _lib.FLAG_STATE_BF16, None)
    assert rc == _lib.GDN_ERR_UNSUPPORTED and 'bf16 states need' in _lib.last_error()
    # no token: the states stay as they are
    q, k, v, g, beta, _ = _inputs(2, 1, 2, 4, 128, torch.bfloat16, seed=1)
    h0 = torch.randn(2, 4, 128, 128, device=dev).bfloat16()
    keep = h0.clone()
    e = lambda x: x[:, :0].to(dev)
    o, ht = _ops()(e(q), e(k), e(v), e(g), beta=e(beta), initial_state=h0, inplace_final_state=True)
    assert o.shape == (2, 0, 4, 128) and torch.equal(ht, keep)


@pytest.mark.parametrize('N,HV,D,vfirst', [(65, 32, 128, False), (67, 32, 128, True), (75, 32, 64, False), (69, 32, 32, False)])
def test_workgroup_placement_with_sequence_counts_that_are_not_multiples_of_8(N, HV, D, vfirst):
    """Launches of 2048 or more workgroups hand every XCD runs of consecutive states; the grid is rounded up to whole
    rounds of 8 runs and the surplus workgroups must do nothing: every state is updated exactly once."""
    H = 8
    q, k, v, g, beta, _ = _inputs(N, 1, H, HV, D, torch.bfloat16, seed=23)
    gen = torch.Generator().manual_seed(24)
    h0 = torch.randn(N, HV, D, D, generator=gen)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, use_qk_l2norm_in_kernel=True)
    dev = 'cuda'
    dh0 = (h0.transpose(-1, -2).contiguous() if vfirst else h0).to(dev)
    o, ht = _ops()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta=beta.to(dev), initial_state=dh0, output_final_state=True,
                   use_qk_l2norm_in_kernel=True, state_v_first=vfirst)
    _check('o', ref_o, o, 5e-3)
    _check('ht', ref_ht, ht.transpose(-1, -2) if vfirst else ht)


@pytest.mark.parametrize('H,HV,D,N,K_prefill', [(2, 4, 128, 8, 128), (8, 32, 128, 40, 256)])
def test_decode_and_prefill_replay_from_a_captured_graph(H, HV, D, N, K_prefill):
    """Serving loops replay captured graphs: the entry points only enqueue kernels on the given
    stream (no allocation, no memset, no synchronisation of their own), so a captured decode step
    and a captured prefill reproduce the eager results on every replay, with eager work and
    synchronisations in between.  (Second case: the decode kernel of the common shape with its placement
    on the XCDs, and the wide-key prefill kernel.)"""
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    dev = 'cuda'
    q, k, v, g, beta, h0 = _inputs(N, 1, H, HV, D, torch.bfloat16, seed=5)
    dq, dk, dv, dg, db = (x.to(dev) for x in (q, k, v, g, beta))
    state = h0.to(dev).contiguous()
    eager_state = state.clone()
    pq, pk, pv, pg, pb, ph = (x.to(dev) for x in O.make_inputs(1, 700, 2, 4, K_prefill, D, seed=6, gate_div=8.0, h0_std=0.5, dtype=torch.bfloat16))
    # warm up outside the capture (library load, kernel attributes)
    _ops()(dq, dk, dv, dg, beta=db, initial_state=state.clone(), output_final_state=True, inplace_final_state=True)
    po_eager, ph_eager = chunk_gated_delta_rule(pq, pk, pv, pg, pb, initial_state=ph, output_final_state=True)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_static, _ = _ops()(dq, dk, dv, dg, beta=db, initial_state=state, output_final_state=True, inplace_final_state=True)
        po_static, ph_static = chunk_gated_delta_rule(pq, pk, pv, pg, pb, initial_state=ph, output_final_state=True)
    state.copy_(h0.to(dev))                      # (the capture itself did not run anything)
    for step in range(3):
        graph.replay()
        o_eager, _ = _ops()(dq, dk, dv, dg, beta=db, initial_state=eager_state, output_final_state=True, inplace_final_state=True)
        torch.cuda.synchronize()
        assert torch.equal(o_static, o_eager), f'decode output differs on replay {step}'
        assert torch.equal(state, eager_state), f'decode state differs on replay {step}'
        assert not torch.isnan(po_eager).any()
        assert torch.equal(po_static, po_eager) and torch.equal(ph_static, ph_eager), f'prefill differs on replay {step}'
        po_static.zero_(); ph_static.zero_()     # the next replay has to write everything again


def test_host_validation_errors():
    op = _ops()
    dev = 'cuda'
    q = torch.randn(2, 4, 2, 64, device=dev)
    v = torch.randn(2, 4, 4, 64, device=dev)
    g = torch.zeros(2, 4, 4, device=dev)
    with pytest.raises(ValueError):
        op(q, q, v, g, cu_seqlens=torch.tensor([0, 4, 8], device=dev))          # batch must be 1
    with pytest.raises(ValueError):
        op(q[:1], q[:1], v[:1], g[:1], initial_state=torch.zeros(3, 4, 64, 64, device=dev),
           cu_seqlens=torch.tensor([0, 2, 4], device=dev))                       # len(h0) != N
    with pytest.raises(ValueError):
        op(q, q, v, g, allow_neg_eigval=True)
    with pytest.raises(ValueError):
        op(q, q, v, g, use_gate_in_kernel=True)
    with pytest.raises(ValueError):
        op(q, q, v, g, state_v_first=True, transpose_state_layout=True)
    with pytest.raises(RuntimeError):
        op(q.cpu(), q.cpu(), v.cpu(), g.cpu())                                   # no CPU path
