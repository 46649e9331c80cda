"""Pins the CPU oracle (oracle/gdn_oracle.py) without running the reference:
scalar fixtures, closed forms, library routines and algebraic invariants.
Each check is chosen so that a plausible slip (dropped term, wrong sign/index,
transposed operand, swapped g/beta) fails it."""
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

GOLD = np.load(os.path.join(os.path.dirname(__file__), 'golden', 'gdn_scalar_cases.npz'))
CASES = ['single_T5', 'gva_T70_h0', 'varlen_h0']


def _gold(name):
    t = lambda key: torch.from_numpy(GOLD[f'{name}.{key}'])
    cu = GOLD[f'{name}.cu'].tolist()
    h0 = t('h0') if f'{name}.h0' in GOLD.files else None
    return dict(q=t('q')[None], k=t('k')[None], v=t('v')[None], g=t('g')[None], beta=t('beta')[None],
                h0=h0, cu=cu, scale=float(GOLD[f'{name}.scale']), o=t('o')[None], ht=t('ht'))


@pytest.mark.parametrize('name', CASES)
def test_recurrent_matches_scalar_fixture(name):
    c = _gold(name)
    o, ht = O.recurrent_gated_delta_rule(c['q'], c['k'], c['v'], c['g'], c['beta'], c['scale'], c['h0'], True,
                                         cu_seqlens=c['cu'], dtype=torch.float64)
    assert torch.allclose(o, c['o'], atol=1e-12, rtol=1e-10)
    assert torch.allclose(ht, c['ht'], atol=1e-12, rtol=1e-10)


@pytest.mark.parametrize('name', CASES)
@pytest.mark.parametrize('chunk', [16, 64])
def test_chunk_matches_scalar_fixture(name, chunk):
    c = _gold(name)
    o, ht = O.chunk_gated_delta_rule(c['q'], c['k'], c['v'], c['g'], c['beta'], c['scale'], c['h0'], True,
                                     cu_seqlens=c['cu'], chunk_size=chunk, dtype=torch.float64)
    # RCP_LN2 is the reference's fp32-rounded 1/ln2 (relative error 1.3e-8 in every exponent)
    assert torch.allclose(o, c['o'], atol=1e-6, rtol=1e-6)
    assert torch.allclose(ht, c['ht'], atol=1e-6, rtol=1e-6)


GOLD_EXT = np.load(os.path.join(os.path.dirname(__file__), 'golden', 'gdn_scalar_cases_ext.npz'))


def _ext(name, key):
    return torch.from_numpy(GOLD_EXT[f'{name}.{key}']) if f'{name}.{key}' in GOLD_EXT.files else None


@pytest.mark.parametrize('name', ['gk_gv_vbeta', 'gk_only_varlen', 'gv_vbeta_varlen'])
def test_optional_decays_and_vector_beta_match_scalar_fixture(name):
    # pins the gk / gv / beta-per-value-column branches of the oracle against the independent scalar loop
    b1 = lambda x: None if x is None else x[None]
    o, ht = O.recurrent_gated_delta_rule(
        b1(_ext(name, 'q')), b1(_ext(name, 'k')), b1(_ext(name, 'v')), b1(_ext(name, 'g')), b1(_ext(name, 'beta')),
        float(GOLD_EXT[f'{name}.scale']), _ext(name, 'h0'), True, cu_seqlens=GOLD_EXT[f'{name}.cu'].tolist(),
        gk=b1(_ext(name, 'gk')), gv=b1(_ext(name, 'gv')), dtype=torch.float64)
    assert torch.allclose(o[0], _ext(name, 'o'), atol=1e-12, rtol=1e-10)
    assert torch.allclose(ht, _ext(name, 'ht'), atol=1e-12, rtol=1e-10)
    # a slip that swaps gk and gv (or drops one) must not pass: the fixture has K != V or only one of them
    assert _ext(name, 'gk') is None or _ext(name, 'gv') is None or _ext(name, 'gk').shape != _ext(name, 'gv').shape


def test_kda_recurrence_matches_scalar_fixture():
    # the KDA operator's recurrence is the token recurrence with a decay per key feature and no scalar gate: the fixture
    # of that form, from the independent scalar loop
    name = 'gk_only_varlen'
    assert _ext(name, 'g') is None and _ext(name, 'gv') is None
    b1 = lambda x: x[None]
    o, ht = O.recurrent_kda(b1(_ext(name, 'q')), b1(_ext(name, 'k')), b1(_ext(name, 'v')), b1(_ext(name, 'gk')), b1(_ext(name, 'beta')),
                            float(GOLD_EXT[f'{name}.scale']), _ext(name, 'h0'), True, cu_seqlens=GOLD_EXT[f'{name}.cu'].tolist(),
                            dtype=torch.float64)
    assert torch.allclose(o[0], _ext(name, 'o'), atol=1e-12, rtol=1e-10)
    assert torch.allclose(ht, _ext(name, 'ht'), atol=1e-12, rtol=1e-10)


def test_kda_gate_pins():
    """Values that the two gate formulas fix (fla/ops/kda/gate.py:27-94), chosen so that a wrong sign, a bias added
    after the activation, A applied outside the sigmoid or a bias indexed [K][HV] instead of [HV][K] fails."""
    HV, K = 2, 3
    z = torch.zeros(1, 1, HV, K)
    A = torch.tensor([0.0, math.log(2.0)])
    # softplus form: -e^A ln 2 at zero input; head 1 decays twice as fast; ~ -e^A x for large x
    out = O.kda_gate(z, A)
    assert torch.allclose(out[0, 0, 0], torch.full((K,), -math.log(2.0))) and torch.allclose(out[0, 0, 1], torch.full((K,), -2 * math.log(2.0)))
    assert torch.allclose(O.kda_gate(z + 30.0, A)[0, 0, :, 0], torch.tensor([-30.0, -60.0]), atol=1e-5)
    assert (O.kda_gate(torch.randn(2, 5, HV, K), A) < 0).all()
    # the bias is added before the activation and is laid out [HV][K]
    bias = torch.zeros(HV * K)
    bias[1 * K + 2] = 30.0                      # head 1, key feature 2
    out = O.kda_gate(z, A, bias)
    assert abs(float(out[0, 0, 1, 2]) + 60.0) < 1e-4
    rest = out.clone(); rest[0, 0, 1, 2] = O.kda_gate(z, A)[0, 0, 1, 2]
    assert torch.equal(rest, O.kda_gate(z, A))
    # without A_log the kernel's constant is exp(1)
    assert torch.allclose(O.kda_gate(z), torch.full((1, 1, HV, K), -math.e * math.log(2.0)))
    # bounded form: lower_bound / 2 at zero input, A multiplies inside the sigmoid, the bound is reached for large inputs
    lb = -5.0
    assert torch.allclose(O.kda_gate(z, A, None, lb), torch.full((1, 1, HV, K), lb / 2))
    out = O.kda_gate(z + 1.0, torch.tensor([0.0, math.log(3.0)]), None, lb)
    assert torch.allclose(out[0, 0, :, 0], torch.tensor([lb / (1 + math.exp(-1.0)), lb / (1 + math.exp(-3.0))]))
    assert torch.allclose(O.kda_gate(z + 40.0, None, None, lb), torch.full((1, 1, HV, K), lb))
    assert torch.allclose(O.kda_gate(z - 40.0, None, None, lb), torch.zeros(1, 1, HV, K), atol=1e-6)
    out = O.kda_gate(z, None, bias, lb)
    assert abs(float(out[0, 0, 1, 2]) - lb) < 1e-6 and abs(float(out[0, 0, 0, 2]) - lb / 2) < 1e-6


def test_pooled_states_of_speculative_decoding_match_scalar_fixture():
    n = 'spec_pool'
    o, pool_after, _ = O.recurrent_gated_delta_rule_pooled(
        _ext(n, 'q')[None], _ext(n, 'k')[None], _ext(n, 'v')[None], _ext(n, 'g')[None], _ext(n, 'beta')[None],
        float(GOLD_EXT[f'{n}.scale']), _ext(n, 'pool'), _ext(n, 'idx'), _ext(n, 'accepted'),
        cu_seqlens=GOLD_EXT[f'{n}.cu'].tolist(), dtype=torch.float64)
    assert torch.allclose(o[0], _ext(n, 'o'), atol=1e-12, rtol=1e-10)
    assert torch.allclose(pool_after, _ext(n, 'pool_after'), atol=1e-12, rtol=1e-10)
    # slots nobody names keep their contents; named ones changed
    named = set(_ext(n, 'idx').flatten().tolist())
    lens = np.diff(GOLD_EXT[f'{n}.cu'])
    written = {int(_ext(n, 'idx')[i, t]) for i in range(len(lens)) for t in range(lens[i])}
    for slot in range(_ext(n, 'pool').shape[0]):
        same = torch.equal(pool_after[slot], _ext(n, 'pool')[slot])
        assert same == (slot not in written), (slot, slot in named)


def test_pooled_one_slot_per_sequence_equals_plain_call():
    q, k, v, g, beta, h0 = O.make_inputs(3, 4, 1, 2, 4, 4, seed=5, h0_std=1.0, N=7)
    idx = torch.tensor([5, 0, 3])
    o, pool_after, per_tok = O.recurrent_gated_delta_rule_pooled(q, k, v, g, beta, None, h0, idx)
    o2, ht2 = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0[idx], True)
    assert torch.allclose(o, o2, atol=1e-6) and torch.allclose(pool_after[idx], ht2, atol=1e-6)
    assert torch.allclose(per_tok.view(3, 4, 2, 4, 4)[:, -1], ht2, atol=1e-6)
    keep = [i for i in range(7) if i not in idx.tolist()]
    assert torch.equal(pool_after[keep], h0[keep])


def test_config1_recurrent_equals_chunk():
    # the CPU-runnable configuration: B=2 T=256 H=2 K=V=64 fp32, zero initial state
    q, k, v, g, beta, _ = O.make_inputs(2, 256, 2, 2, 64, 64, seed=42)
    o_r, h_r = O.recurrent_gated_delta_rule(q, k, v, g, beta, output_final_state=True)
    o_c, h_c = O.chunk_gated_delta_rule(q, k, v, g, beta, output_final_state=True)
    assert h_r.shape == (2, 2, 64, 64)
    assert O.get_err_ratio(o_r, o_c) < 1e-4 and O.get_err_ratio(h_r, h_c) < 1e-4
    o_d, h_d = O.chunk_gated_delta_rule(q, k, v, g, beta, output_final_state=True, dtype=torch.float64)
    assert O.get_err_ratio(o_d, o_c) < 1e-5 and O.get_err_ratio(h_d, h_r) < 1e-5


def test_one_step_closed_forms():
    torch.manual_seed(0)
    N, H, HV, K, V = 3, 2, 4, 8, 5
    q = torch.randn(N, H, K, dtype=torch.float64)
    k = F.normalize(torch.randn(N, H, K, dtype=torch.float64), dim=-1)
    v = torch.randn(N, HV, V, dtype=torch.float64)
    S = torch.randn(N, HV, K, V, dtype=torch.float64)
    g = -torch.rand(N, HV, dtype=torch.float64)
    beta = torch.rand(N, HV, dtype=torch.float64)
    call = lambda g_, b_: O.recurrent_gated_delta_rule(q[:, None], k[:, None], v[:, None], g_[:, None], b_[:, None],
                                                        1.0, S, True, dtype=torch.float64)
    # beta = 0: pure decay, output reads the decayed state
    o, S1 = call(g, torch.zeros_like(beta))
    Sd = S * g.exp()[:, :, None, None]
    assert torch.allclose(S1, Sd)
    assert torch.allclose(o[:, 0], torch.einsum('nhkv,nhk->nhv', Sd, q.repeat_interleave(2, 1)))
    # g = 0, beta = 1, |k| = 1: the state is overwritten so that S'^T k = v exactly
    o, S1 = call(torch.zeros_like(g), torch.ones_like(beta))
    assert torch.allclose(torch.einsum('nhkv,nhk->nhv', S1, k.repeat_interleave(2, 1)), v)
    # general closed form  S' = e^g S + k [beta (v - e^g S^T k)]^T
    o, S1 = call(g, beta)
    kk = k.repeat_interleave(2, 1)
    d = beta[..., None] * (v - torch.einsum('nhkv,nhk->nhv', Sd, kk))
    assert torch.allclose(S1, Sd + kk[..., None] * d[:, :, None, :])
    # decode_step helper is the same map (fp32)
    o32, S32 = O.decode_step(q, k, v, g, beta, S, scale=1.0)
    assert torch.allclose(S32.double(), S1, atol=1e-5) and torch.allclose(o32.double(), o[:, 0], atol=1e-5)


def test_argument_order_is_g_then_beta_for_chunk():
    # swapping g and beta must change the result (guards the (beta, g) vs (g, beta) slip)
    q, k, v, g, beta, _ = O.make_inputs(1, 40, 1, 1, 4, 4, seed=3)
    o1, _ = O.chunk_gated_delta_rule(q, k, v, g, beta)
    o2, _ = O.chunk_gated_delta_rule(q, k, v, beta, g)
    assert O.get_err_ratio(o1, o2) > 1e-2


def test_T_steps_equal_chained_single_steps_and_split_handoff():
    q, k, v, g, beta, h0 = O.make_inputs(2, 150, 2, 4, 16, 8, seed=5, h0_std=0.3)
    o, ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True, dtype=torch.float64)
    S = h0.double()
    for t in range(150):
        o_t, S = O.recurrent_gated_delta_rule(q[:, t:t + 1], k[:, t:t + 1], v[:, t:t + 1], g[:, t:t + 1], beta[:, t:t + 1],
                                              initial_state=S, output_final_state=True, dtype=torch.float64)
        assert torch.allclose(o_t[:, 0], o[:, t], atol=1e-12)
    assert torch.allclose(S, ht, atol=1e-12)
    # chunk op: split T at a non-multiple of the chunk size, hand the state over
    oc, hc = O.chunk_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True, dtype=torch.float64)
    o1, h1 = O.chunk_gated_delta_rule(q[:, :70], k[:, :70], v[:, :70], g[:, :70], beta[:, :70], initial_state=h0,
                                      output_final_state=True, dtype=torch.float64)
    o2, h2 = O.chunk_gated_delta_rule(q[:, 70:], k[:, 70:], v[:, 70:], g[:, 70:], beta[:, 70:], initial_state=h1,
                                      output_final_state=True, dtype=torch.float64)
    assert torch.allclose(torch.cat([o1, o2], 1), oc, atol=1e-10) and torch.allclose(h2, hc, atol=1e-10)
    assert torch.allclose(oc, o, atol=1e-10) and torch.allclose(hc, ht, atol=1e-10)


def test_varlen_equals_per_sequence_loop_and_gva_equals_repeat():
    cu = [0, 15, 100, 300, 301, 520]
    q, k, v, g, beta, h0 = O.make_inputs(1, 520, 2, 4, 8, 8, seed=7, h0_std=0.5, N=5)
    for fn in (O.recurrent_gated_delta_rule, O.chunk_gated_delta_rule):
        o, ht = fn(q, k, v, g, beta, initial_state=h0, output_final_state=True, cu_seqlens=cu, dtype=torch.float64)
        for n, (s, e) in enumerate(zip(cu[:-1], cu[1:])):
            o_n, h_n = fn(q[:, s:e], k[:, s:e], v[:, s:e], g[:, s:e], beta[:, s:e], initial_state=h0[n:n + 1],
                          output_final_state=True, dtype=torch.float64)
            assert torch.equal(o_n[0], o[0, s:e]) and torch.equal(h_n[0], ht[n])
        qe, ke = q.repeat_interleave(2, 2), k.repeat_interleave(2, 2)
        o_e, h_e = fn(qe, ke, v, g, beta, initial_state=h0, output_final_state=True, cu_seqlens=cu, dtype=torch.float64)
        assert torch.equal(o_e, o) and torch.equal(h_e, ht)


def test_state_v_first_is_a_transpose():
    q, k, v, g, beta, h0 = O.make_inputs(2, 70, 1, 2, 8, 4, seed=9, h0_std=0.5)
    for fn in (O.recurrent_gated_delta_rule, O.chunk_gated_delta_rule):
        o, ht = fn(q, k, v, g, beta, initial_state=h0, output_final_state=True)
        o2, ht2 = fn(q, k, v, g, beta, initial_state=h0.transpose(-1, -2).contiguous(), output_final_state=True,
                     state_v_first=True)
        assert ht2.shape == (2, 2, 4, 8)
        assert torch.equal(o, o2) and torch.equal(ht2.transpose(-1, -2), ht)


def test_stages_solve_wy_and_scan_invariants():
    q, k, v, g, beta, h0 = O.make_inputs(1, 150, 1, 2, 16, 8, seed=11, h0_std=0.5)
    o, ht, st = O.chunk_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True,
                                         dtype=torch.float64, return_stages=True)
    st = st[0]
    assert [x.shape[-1] for x in st['G']] == [64, 64, 22]           # tail chunk is the leading r x r problem
    kk = k.double().repeat_interleave(2, 2)[0]
    for c, (L, A, G, w, u) in enumerate(zip(st['L'], st['A'], st['G'], st['w'], st['u'])):
        r = L.shape[-1]
        eye = torch.eye(r, dtype=torch.float64)
        # library routine + definition: A (I+L) = I, unit lower triangular
        assert torch.allclose(A, torch.linalg.inv(eye + L), atol=1e-10)
        assert torch.allclose(A @ (eye + L), eye.expand_as(A), atol=1e-10)
        assert torch.equal(A.triu(1), torch.zeros_like(A)) and torch.allclose(A.diagonal(dim1=-2, dim2=-1), torch.ones(2, r, dtype=torch.float64))
        assert torch.equal(L.triu(0), torch.zeros_like(L))
        # the row-by-row substitution of naive.py:129-131 gives the same inverse
        attn = -L.clone()
        for i in range(1, r):
            attn[..., i, :i] = attn[..., i, :i] + (attn[..., i, :i, None] * attn[..., :i, :i]).sum(-2)
        assert torch.allclose(attn + eye, A, atol=1e-10)
        # cumsum closed form, restarted per chunk, in log2 units
        gc = g[0, c * 64:c * 64 + r].double().transpose(0, 1)
        assert torch.allclose(G, gc.cumsum(-1) / math.log(2), atol=1e-6)
        # w,u plain definitions
        b = beta[0, c * 64:c * 64 + r].double().transpose(0, 1)
        kc = kk[c * 64:c * 64 + r].transpose(0, 1)
        vc = v[0, c * 64:c * 64 + r].double().transpose(0, 1)
        assert torch.allclose(u, A @ (vc * b[..., None]), atol=1e-12)
        assert torch.allclose(w, A @ (kc * (b * torch.exp2(G))[..., None]), atol=1e-12)
    assert torch.equal(st['h'][0], h0[0].double())                   # h[0] == h0
    cs = O.chunk_local_cumsum(g, 64, scale=O.RCP_LN2)
    assert torch.allclose(cs[0, :64].double(), st['G'][0].transpose(0, 1), atol=1e-5)
    rev = O.chunk_local_cumsum(g, 64, reverse=True)
    assert torch.allclose(rev[0, 128:150], g[0, 128:150].flip(0).cumsum(0).flip(0), atol=1e-6)


def test_flags_equal_host_side_prologues():
    torch.manual_seed(1)
    B, T, H, HV, K, V = 1, 70, 2, 4, 8, 8
    q, k, v = torch.randn(B, T, H, K), torch.randn(B, T, H, K), torch.randn(B, T, HV, V)
    graw, braw = torch.randn(B, T, HV), torch.randn(B, T, HV)
    A_log, dt_bias = torch.randn(HV) * 0.3, torch.randn(HV) * 0.3
    for fn in (O.recurrent_gated_delta_rule, O.chunk_gated_delta_rule):
        o1, h1 = fn(q, k, v, graw, braw, output_final_state=True, use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True,
                    A_log=A_log, dt_bias=dt_bias, use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True)
        gd = -A_log.exp() * F.softplus(graw + dt_bias)
        o2, h2 = fn(O.l2norm(q), O.l2norm(k), v, gd, 2 * torch.sigmoid(braw), output_final_state=True)
        assert O.get_err_ratio(o2, o1) < 1e-5 and O.get_err_ratio(h2, h1) < 1e-5
    x = torch.randn(5, 7)
    assert torch.allclose(O.l2norm(x), x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6))


def test_index_tables():
    cu = [0, 1, 65, 192, 193, 400]
    idx = O.prepare_chunk_indices(cu, 64)
    assert idx == [[0, 0], [1, 0], [2, 0], [2, 1], [3, 0], [4, 0], [4, 1], [4, 2], [4, 3]]
    assert O.prepare_chunk_offsets(cu, 64) == [0, 1, 2, 4, 5, 9]
    assert O.prepare_chunk_offsets([0, 64], 64) == [0, 1]


def test_error_metric_definition():
    x = torch.tensor([3.0, 4.0]); y = torch.tensor([3.0, 5.0])
    assert abs(O.get_abs_err(x, y) - 1.0) < 1e-12
    assert abs(O.get_err_ratio(x, y) - (math.sqrt(0.5) / (math.sqrt(12.5) + 1e-8))) < 1e-12


def test_varlen_length_recipe():
    L = O.make_varlen_lengths(65536, 32, 256, 4096, seed=42)
    assert len(L) == 32 and sum(L) == 65536 and min(L) >= 1


# --------------------------------------------------------------------------- #
# comba (a second key p for the prediction, taken before the token's decay)
# --------------------------------------------------------------------------- #
def _comba_inputs(B, T, H, K, V, seed, gate_div=1.0):
    gen = torch.Generator().manual_seed(seed)
    q = F.normalize(torch.randn(B, T, H, K, generator=gen, dtype=torch.float64), dim=-1)
    k = F.normalize(torch.randn(B, T, H, K, generator=gen, dtype=torch.float64), dim=-1)
    p = F.normalize(torch.randn(B, T, H, K, generator=gen, dtype=torch.float64), dim=-1)
    v = torch.randn(B, T, H, V, generator=gen, dtype=torch.float64)
    g = F.logsigmoid(torch.rand(B, T, H, generator=gen, dtype=torch.float64)) / gate_div
    beta = torch.rand(B, T, H, generator=gen, dtype=torch.float64).sigmoid()
    h0 = torch.randn(B, H, K, V, generator=gen, dtype=torch.float64)
    return q, k, v, p, g, beta, h0


def test_comba_recurrence_against_scalar_loops():
    """The token recurrence written again as loops over single numbers (fla/ops/comba/fused_recurrent.py:85-105: predict
    with p on the undecayed state, then decay, then write k).  A prediction taken after the decay, or with k, fails it."""
    B, T, H, K, V = 1, 5, 2, 3, 2
    q, k, v, p, g, beta, h0 = _comba_inputs(B, T, H, K, V, seed=3)
    scale = 0.7
    o, ht = O.recurrent_comba(q, k, v, p, g, beta, scale, h0, True, dtype=torch.float64)
    for h in range(H):
        S = [[float(h0[0, h, a, c]) for c in range(V)] for a in range(K)]
        for t in range(T):
            pred = [sum(S[a][c] * float(p[0, t, h, a]) for a in range(K)) for c in range(V)]
            vn = [float(beta[0, t, h]) * (float(v[0, t, h, c]) - pred[c]) for c in range(V)]
            eg = math.exp(float(g[0, t, h]))
            for a in range(K):
                for c in range(V):
                    S[a][c] = eg * S[a][c] + float(k[0, t, h, a]) * vn[c]
            for c in range(V):
                want = scale * sum(S[a][c] * float(q[0, t, h, a]) for a in range(K))
                assert abs(float(o[0, t, h, c]) - want) < 1e-12
        for a in range(K):
            for c in range(V):
                assert abs(float(ht[0, h, a, c]) - S[a][c]) < 1e-12


def test_comba_reductions_and_chunk_form():
    """p = k and g = 0 is the plain delta rule; the chunked form (in-chunk inverse, fla/ops/comba/naive.py:113-160) is the
    same map as the recurrence for every chunk size; l2 norm in the kernel equals normalising q, k and p beforehand."""
    B, T, H, K, V = 2, 150, 2, 16, 12
    q, k, v, p, g, beta, h0 = _comba_inputs(B, T, H, K, V, seed=5, gate_div=0.5)
    zero = torch.zeros_like(g)
    o1, s1 = O.recurrent_comba(q, k, v, None, zero, beta, None, h0, True, dtype=torch.float64)
    o2, s2 = O.recurrent_gated_delta_rule(q, k, v, zero, beta, None, h0, True, dtype=torch.float64)
    assert (o1 - o2).abs().max() < 1e-12 and (s1 - s2).abs().max() < 1e-12
    # with p = k and a decay, comba differs from the gated delta rule only in what the prediction sees: e^-g times it
    o3, _ = O.recurrent_comba(q[:, :1], k[:, :1], v[:, :1], None, g[:, :1], beta[:, :1], 1.0, h0, True, dtype=torch.float64)
    pred = torch.einsum('bhkv,bhk->bhv', h0, k[:, 0])
    S1 = h0 * g[:, 0].exp()[..., None, None] + k[:, 0, :, :, None] * (beta[:, 0, :, None] * (v[:, 0] - pred))[:, :, None, :]
    assert (o3[:, 0] - torch.einsum('bhkv,bhk->bhv', S1, q[:, 0])).abs().max() < 1e-12

    ref_o, ref_s = O.recurrent_comba(q, k, v, p, g, beta, 0.3, h0, True, dtype=torch.float64)
    for chunk in (16, 64):
        for b in range(B):
            for h in range(H):
                oc, sc = O.chunk_comba_one_sequence(q[b, :, h], k[b, :, h], v[b, :, h], p[b, :, h], g[b, :, h], beta[b, :, h],
                                                    0.3, h0[b, h], chunk, torch.float64)
                assert (oc - ref_o[b, :, h]).abs().max() < 1e-10 and (sc - ref_s[b, h]).abs().max() < 1e-10
    raw = [x * 3.0 for x in (q, k, p)]
    o4, s4 = O.recurrent_comba(raw[0], raw[1], v, raw[2], g, beta, 0.3, h0, True, use_qk_l2norm_in_kernel=True, dtype=torch.float64)
    assert (o4 - ref_o).abs().max() < 1e-6 and (s4 - ref_s).abs().max() < 1e-6
    # packed sequences and grouped value heads
    cu = [0, 40, 150]
    qp, kp, vp, pp, gp, bp = (x[:1] for x in (q, k, v, p, g, beta))
    o5, s5 = O.recurrent_comba(qp, kp, vp, pp, gp, bp, 0.3, h0, True, cu_seqlens=cu, dtype=torch.float64)
    for n in range(2):
        sl = slice(cu[n], cu[n + 1])
        on, sn = O.recurrent_comba(qp[:, sl], kp[:, sl], vp[:, sl], pp[:, sl], gp[:, sl], bp[:, sl], 0.3, h0[n:n + 1], True, dtype=torch.float64)
        assert torch.equal(o5[:, sl], on) and torch.equal(s5[n:n + 1], sn)
    o6, _ = O.recurrent_comba(q[:, :, :1], k[:, :, :1], v, p[:, :, :1], g, beta, 0.3, h0, dtype=torch.float64)
    o7, _ = O.recurrent_comba(q[:, :, :1].expand(-1, -1, 2, -1), k[:, :, :1].expand(-1, -1, 2, -1), v, p[:, :, :1].expand(-1, -1, 2, -1),
                              g, beta, 0.3, h0, dtype=torch.float64)
    assert torch.equal(o6, o7)
    # a beta per value column: every column is a recurrence of its own with that column's beta
    bv = torch.rand(B, T, H, V, dtype=torch.float64)
    o8, s8 = O.recurrent_comba(q, k, v, p, g, bv, 0.3, h0, True, dtype=torch.float64)
    for c in (0, V - 1):
        oc, sc = O.recurrent_comba(q, k, v[..., c:c + 1], p, g, bv[..., c], 0.3, h0[..., c:c + 1], True, dtype=torch.float64)
        assert (o8[..., c:c + 1] - oc).abs().max() < 1e-12 and (s8[..., c:c + 1] - sc).abs().max() < 1e-12


@pytest.mark.parametrize('kw', [dict(), dict(use_qk_l2norm_in_kernel=True), dict(cu_seqlens=[0, 4, 11])])
def test_comba_grads_match_finite_differences(kw):
    """``comba_grads`` (reverse mode through the recurrence) against central differences of the recurrence itself, along a
    random direction in every input; grouped value heads, rows that are not unit vectors, an initial state."""
    B, T, H, HV, K, V = (1, 11, 2, 4, 5, 3) if 'cu_seqlens' in kw else (2, 8, 2, 4, 5, 3)
    gen = torch.Generator().manual_seed(11)
    f64 = dict(generator=gen, dtype=torch.float64)
    q, k, p = (torch.randn(B, T, H, K, **f64) * s for s in (1.3, 0.6, 0.9))
    v = torch.randn(B, T, HV, V, **f64)
    g = F.logsigmoid(torch.randn(B, T, HV, **f64))
    beta = torch.rand(B, T, HV, **f64)
    h0 = torch.randn(2, HV, K, V, **f64) * 0.5
    do, dht = torch.randn(B, T, HV, V, **f64), torch.randn(2, HV, K, V, **f64)
    grads = O.comba_grads(q, k, v, p, g, beta, do, dht, scale=0.4, initial_state=h0, **kw)
    inputs = dict(dq=q, dk=k, dv=v, dp=p, dg=g, dbeta=beta, dh0=h0)

    def loss(a):
        o, ht = O.recurrent_comba(a['dq'], a['dk'], a['dv'], a['dp'], a['dg'], a['dbeta'], 0.4, a['dh0'], True, dtype=torch.float64, **kw)
        return float((o * do).sum() + (ht * dht).sum())
    eps = 1e-6
    for name, x in inputs.items():
        d = torch.randn(x.shape, **f64)
        fd = (loss({**inputs, name: x + eps * d}) - loss({**inputs, name: x - eps * d})) / (2 * eps)
        an = float((grads[name] * d).sum())
        assert abs(fd - an) <= 1e-6 * max(1.0, abs(an)), f'{name}: finite difference {fd} vs gradient {an}'


@pytest.mark.parametrize('kw', [
    dict(),
    dict(use_qk_l2norm_in_kernel=True, use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True),
    dict(use_gate_in_kernel=True),
    dict(use_gate_in_kernel=True, lower_bound=-3.0),
    dict(use_gate_in_kernel=True, lower_bound=-3.0, no_A=True),
    dict(cu_seqlens=[0, 4, 11], state_v_first=True),
])
def test_kda_grads_match_finite_differences(kw):
    """``kda_grads`` (reverse mode through the recurrence) against central differences of the recurrence itself, along a
    random direction in every input and gate parameter."""
    kw = dict(kw)
    no_A = kw.pop('no_A', False)
    B, T, H, HV, K, V = (1, 11, 2, 4, 5, 3) if 'cu_seqlens' in kw else (2, 8, 2, 4, 5, 3)
    gen = torch.Generator().manual_seed(13)
    f64 = dict(generator=gen, dtype=torch.float64)
    q, k = torch.randn(B, T, H, K, **f64) * 1.3, torch.randn(B, T, H, K, **f64) * 0.6
    v = torch.randn(B, T, HV, V, **f64)
    gate = kw.get('use_gate_in_kernel', False)
    g = torch.randn(B, T, HV, K, **f64) if gate else F.logsigmoid(torch.randn(B, T, HV, K, **f64))
    beta = torch.randn(B, T, HV, **f64) if kw.get('use_beta_sigmoid_in_kernel') else torch.rand(B, T, HV, **f64)
    h0 = torch.randn(2, HV, V, K, **f64) * 0.5 if kw.get('state_v_first') else torch.randn(2, HV, K, V, **f64) * 0.5
    do, dht = torch.randn(B, T, HV, V, **f64), torch.randn(*h0.shape, **f64)
    inputs = dict(dq=q, dk=k, dv=v, dg=g, dbeta=beta, dh0=h0)
    if gate:
        if not no_A:
            inputs['dA_log'] = torch.randn(HV, **f64) * 0.3
        inputs['ddt_bias'] = torch.randn(HV * K, **f64) * 0.3

    grads = O.kda_grads(q, k, v, g, beta, do, dht, scale=0.4, initial_state=h0, A_log=inputs.get('dA_log'),
                        dt_bias=inputs.get('ddt_bias'), dtype=torch.float64, **kw)

    def loss(a):
        o, ht = O.recurrent_kda(a['dq'], a['dk'], a['dv'], a['dg'], a['dbeta'], scale=0.4, initial_state=a['dh0'],
                                output_final_state=True, A_log=a.get('dA_log'), dt_bias=a.get('ddt_bias'), dtype=torch.float64, **kw)
        return float((o * do).sum() + (ht * dht).sum())
    eps = 1e-6
    for name, x in inputs.items():
        d = torch.randn(x.shape, **f64)
        fd = (loss({**inputs, name: x + eps * d}) - loss({**inputs, name: x - eps * d})) / (2 * eps)
        an = float((grads[name] * d).sum())
        assert abs(fd - an) <= 1e-6 * max(1.0, abs(an)), f'{name}: finite difference {fd} vs gradient {an}'

