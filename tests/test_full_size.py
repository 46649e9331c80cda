"""GPU parity at the full sizes of the benchmark configurations (the inputs bench.py times):
direct comparison with the fp32 CPU oracle where it finishes in seconds, plus properties that do
not depend on the size: exact homogeneity in (v, h0), hand-off of the state between two calls,
and equality of the packed and the per-sequence evaluation."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu

RATIO, MAXABS = 5e-3, 1e-2          # rel-RMSE and max-abs-error ratio vs the fp32 oracle


def _inputs(B, T, H, HV, N=None, h0=True, seed=42, gate_div=16.0):
    gen = torch.Generator().manual_seed(seed)
    q = F.normalize(torch.randn(B, T, H, 128, generator=gen), p=2, dim=-1).bfloat16()
    k = F.normalize(torch.randn(B, T, H, 128, generator=gen), p=2, dim=-1).bfloat16()
    v = torch.randn(B, T, HV, 128, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, HV, generator=gen)) / gate_div
    beta = torch.sigmoid(torch.randn(B, T, HV, generator=gen))
    s = 0.1 * torch.randn(N or B, HV, 128, 128, generator=gen) if h0 else None
    return q, k, v, g, beta, s


def _op():
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    return chunk_gated_delta_rule


def _gpu(*xs):
    return [None if x is None else x.cuda() for x in xs]


def _check(name, ref, got):
    got = got.detach().float().cpu()
    assert got.shape == ref.shape and not torch.isnan(got).any(), name
    r, m = O.get_err_ratio(ref, got), O.max_abs_ratio(ref, got)
    assert r <= RATIO and m <= MAXABS, f'{name}: rel-rmse {r:.3e} max-abs ratio {m:.3e}'


@pytest.mark.parametrize('B,T,H,HV,h0', [(4, 4096, 16, 16, False), (1, 32768, 16, 32, True)])
def test_dense_configurations_against_the_oracle(B, T, H, HV, h0):
    q, k, v, g, beta, s = _inputs(B, T, H, HV, h0=h0)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, s, True)
    dq, dk, dv, dg, db, ds = _gpu(q, k, v, g, beta, s)
    o, ht = _op()(dq, dk, dv, dg, db, initial_state=ds, output_final_state=True)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


def test_long_sequence_properties():
    """B=1, T=32768, 16 q/k heads, 32 value heads (evaluated in time segments)."""
    q, k, v, g, beta, s = _inputs(1, 32768, 16, 32)
    dq, dk, dv, dg, db, ds = _gpu(q, k, v, g, beta, s)
    op = _op()
    o, ht = op(dq, dk, dv, dg, db, initial_state=ds, output_final_state=True)
    # (1) o and the final state are linear in (v, h0); scaling both by a power of two commutes with every
    # rounding on the way (nothing overflows or underflows here), so the result scales bit for bit
    o2, ht2 = op(dq, dk, dv * 2, dg, db, initial_state=ds * 2, output_final_state=True)
    assert torch.equal(o2, o * 2) and torch.equal(ht2, ht * 2)
    # (2) the state handed from one call to the next: two halves reproduce the whole up to rounding
    # (the halves are cut into different segments than the whole)
    h = 32768 // 2 + 64 * 3 + 17                         # not on a chunk boundary
    oa, sa = op(dq[:, :h], dk[:, :h], dv[:, :h], dg[:, :h], db[:, :h], initial_state=ds, output_final_state=True)
    ob, sb = op(dq[:, h:], dk[:, h:], dv[:, h:], dg[:, h:], db[:, h:], initial_state=sa, output_final_state=True)
    _check('o (two calls)', o.float().cpu(), torch.cat([oa, ob], 1))
    _check('ht (two calls)', ht.float().cpu(), sb)
    # (3) every other form of the sequential stage agrees with the automatic choice: a single pass over
    # the sequence, and segments with one or two runs per workgroup throughout
    import os
    for mode in ('wide-single', 'wide-pair', 'segments-single', 'segments-exact-single', 'segments-pair'):
        os.environ['FLA_HIP_SCAN_MODE'] = mode
        try:
            ow, hw = op(dq, dk, dv, dg, db, initial_state=ds, output_final_state=True)
        finally:
            del os.environ['FLA_HIP_SCAN_MODE']
        _check(f'o ({mode})', o.float().cpu(), ow)
        _check(f'ht ({mode})', ht.float().cpu(), hw)


def test_packed_65536_tokens_in_32_sequences():
    lens = O.make_varlen_lengths(65536, 32, 256, 4096, seed=42)
    cu = [0]
    for x in lens:
        cu.append(cu[-1] + x)
    q, k, v, g, beta, s = _inputs(1, 65536, 16, 32, N=32)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, s, True, cu_seqlens=cu)
    dq, dk, dv, dg, db, ds = _gpu(q, k, v, g, beta, s)
    cu_t = torch.tensor(cu, dtype=torch.int64, device='cuda')
    o, ht = _op()(dq, dk, dv, dg, db, initial_state=ds, output_final_state=True, cu_seqlens=cu_t)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    # the three longest and the shortest sequence, each alone
    order = sorted(range(32), key=lambda i: -lens[i])
    for n in order[:3] + order[-1:]:
        a, b = cu[n], cu[n + 1]
        on, hn = _op()(dq[:, a:b], dk[:, a:b], dv[:, a:b], dg[:, a:b], db[:, a:b], initial_state=ds[n:n + 1], output_final_state=True)
        _check(f'o[{n}] alone', o[0, a:b].float().cpu(), on[0])
        _check(f'ht[{n}] alone', ht[n].float().cpu(), hn[0])


def test_decode_batch_256_against_the_oracle_and_chained():
    from fla_hip.ops.gated_delta_rule import fused_recurrent_gated_delta_rule as rec
    N, H, HV = 256, 16, 32
    gen = torch.Generator().manual_seed(42)
    q = F.normalize(torch.randn(N, 2, H, 128, generator=gen), p=2, dim=-1).bfloat16()
    k = F.normalize(torch.randn(N, 2, H, 128, generator=gen), p=2, dim=-1).bfloat16()
    v = torch.randn(N, 2, HV, 128, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(N, 2, HV, generator=gen))
    beta = torch.sigmoid(torch.randn(N, 2, HV, generator=gen))
    s0 = 0.1 * torch.randn(N, HV, 128, 128, generator=gen)
    S = s0.clone()
    refs = []
    for t in range(2):
        o_ref, S = O.decode_step(q[:, t], k[:, t], v[:, t], g[:, t], beta[:, t], S)
        refs.append(o_ref)
    dq, dk, dv, dg, db = _gpu(q, k, v, g, beta)
    pool = s0.cuda()
    for t in range(2):                                   # two single-token steps on the state pool, in place
        o, pool2 = rec(dq[:, t:t + 1], dk[:, t:t + 1], dv[:, t:t + 1], dg[:, t:t + 1], beta=db[:, t:t + 1],
                       initial_state=pool, output_final_state=True, inplace_final_state=True)
        assert pool2.data_ptr() == pool.data_ptr()
        r = O.get_err_ratio(refs[t].float(), o[:, 0].float().cpu())
        assert r <= 2e-3, f'o step {t}: {r:.3e}'
    assert O.get_err_ratio(S, pool.cpu()) <= 2e-3
    # the same two tokens in one call
    o12, s12 = rec(dq, dk, dv, dg, beta=db, initial_state=s0.cuda(), output_final_state=True)
    assert O.get_err_ratio(S, s12.cpu()) <= 2e-3
