"""GPU parity of chunk_gated_delta_rule for wide keys, 128 < K <= 256 (the reference's scan covers K <= 256 on its chunk
path: fla/ops/common/chunk_delta_h.py:108-114, assert :712; its layer defaults to head_dim 256 with twice as many value
columns: fla/layers/gated_deltanet.py:91-92), against the fp32 CPU oracle on the same seeded inputs.  These shapes run the
wide-key scan kernel: 64 value columns per workgroup, any number of value columns per head."""
import pytest
import torch

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu

# o and final state: relative RMSE <= 5e-3 and max-abs-error ratio <= 1e-2 vs the fp32 oracle
RATIO, MAXABS = 5e-3, 1e-2


def _op():
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    return chunk_gated_delta_rule


def _check(name, ref, got, ratio=RATIO):
    got = got.detach().float().cpu()
    assert got.shape == ref.shape, f'{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}'
    assert not torch.isnan(got).any(), f'{name}: NaN'
    r, m = O.get_err_ratio(ref, got), O.max_abs_ratio(ref, got)
    assert r <= ratio and m <= MAXABS, f'{name}: rel-rmse {r:.3e} max-abs ratio {m:.3e}'


def _run(q, k, v, g, beta, h0=None, cu=None, **kw):
    dev = 'cuda'
    cu_t = None if cu is None else torch.tensor(cu, dtype=kw.pop('idx_dtype', torch.int64), device=dev)
    return _op()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta.to(dev),
                 initial_state=None if h0 is None else h0.to(dev), output_final_state=True, cu_seqlens=cu_t, **kw)


@pytest.mark.parametrize('B,T,H,HV,K,V,gate_div,with_h0,dtype', [
    (2, 1024, 4, 4, 256, 256, 16.0, False, torch.bfloat16),
    (1, 2048, 2, 4, 256, 512, 16.0, True, torch.bfloat16),     # the layer's default head: K = 256, V = 512, grouped values
    (1, 64, 1, 1, 256, 64, 1.0, False, torch.bfloat16),        # one chunk, one workgroup
    (2, 63, 1, 2, 256, 128, 1.0, True, torch.bfloat16),        # shorter than a chunk
    (1, 1000, 2, 2, 256, 128, 4.0, True, torch.float16),       # f16: the state is rescaled every chunk
    (2, 333, 3, 6, 136, 72, 2.0, True, torch.bfloat16),        # just above 128, value columns past the block
    (1, 500, 2, 4, 192, 200, 8.0, True, torch.bfloat16),
    (1, 200, 1, 1, 250, 100, 1.0, True, torch.bfloat16),       # not multiples of 8: padded on the host
    (1, 130, 9, 9, 256, 64, 1.0, False, torch.bfloat16),       # more (sequence, q/k head) groups than one round of 8 XCDs
])
def test_wide_keys_vs_oracle(B, T, H, HV, K, V, gate_div, with_h0, dtype):
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, K, V, seed=42, gate_div=gate_div,
                                         h0_std=0.5 if with_h0 else None, dtype=dtype)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    o, ht = _run(q, k, v, g, beta, h0)
    assert o.dtype == q.dtype and ht.dtype == torch.float32 and o.shape == (B, T, HV, V)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('cu,H,HV,K,V', [
    ([0, 1024, 2048], 4, 4, 256, 256),
    ([0, 15], 2, 2, 256, 64),
    ([0, 1, 100, 101, 300, 1200, 2048], 2, 4, 256, 512),
    ([0, 64, 65, 700], 1, 2, 160, 96),
])
@pytest.mark.parametrize('idx_dtype', [torch.int64, torch.int32])
def test_wide_keys_packed_and_bit_exact_ownership(cu, H, HV, K, V, idx_dtype):
    T, N = cu[-1], len(cu) - 1
    q, k, v, g, beta, h0 = O.make_inputs(1, T, H, HV, K, V, seed=11, gate_div=2.0, h0_std=0.5, N=N, dtype=torch.bfloat16)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu_seqlens=cu)
    o, ht = _run(q, k, v, g, beta, h0, cu, idx_dtype=idx_dtype)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    # every sequence run alone through the same kernels reproduces the packed result bit for bit
    for n, (s, e) in enumerate(zip(cu[:-1], cu[1:])):
        o_n, h_n = _run(q[:, s:e], k[:, s:e], v[:, s:e], g[:, s:e], beta[:, s:e], h0[n:n + 1])
        assert torch.equal(o_n[0], o[0, s:e]), f'sequence {n}: o differs'
        assert torch.equal(h_n[0], ht[n]), f'sequence {n}: state differs'


def test_wide_keys_prologues_and_state_layout():
    """In-kernel l2 norm, gate activation, beta sigmoid with negative eigenvalues and the V-first state layout, all at once,
    on unnormalised q and k (fla/ops/gated_delta_rule/chunk.py:278-288, :510-540)."""
    B, T, H, HV, K, V = 2, 400, 2, 4, 256, 192
    gen = torch.Generator().manual_seed(3)
    q, k = torch.randn(B, T, H, K, generator=gen).bfloat16(), torch.randn(B, T, H, K, generator=gen).bfloat16()
    v = torch.randn(B, T, HV, V, generator=gen).bfloat16()
    g, beta = torch.randn(B, T, HV, generator=gen), torch.randn(B, T, HV, generator=gen)
    A_log, dt_bias = 0.3 * torch.randn(HV, generator=gen), 0.3 * torch.randn(HV, generator=gen)
    h0 = 0.5 * torch.randn(B, HV, K, V, generator=gen)
    kw = dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True, use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, A_log=A_log, dt_bias=dt_bias, **kw)
    o, ht = _run(q, k, v, g, beta, h0.transpose(-1, -2).contiguous(), state_v_first=True, A_log=A_log.cuda(), dt_bias=dt_bias.cuda(), **kw)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht.transpose(-1, -2))


def test_wide_keys_chained_calls_and_decode_handoff():
    """Two calls chained through the state equal one call; the state then continues in the token recurrence."""
    from fla_hip.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    B, T, H, HV, K, V = 1, 640, 2, 2, 256, 128
    q, k, v, g, beta, h0 = O.make_inputs(B, T + 4, H, HV, K, V, seed=8, gate_div=4.0, h0_std=0.5, dtype=torch.bfloat16)
    cut = 256
    o_all, h_all = _run(q[:, :T], k[:, :T], v[:, :T], g[:, :T], beta[:, :T], h0)
    o_a, h_a = _run(q[:, :cut], k[:, :cut], v[:, :cut], g[:, :cut], beta[:, :cut], h0)
    o_b, h_b = _run(q[:, cut:T], k[:, cut:T], v[:, cut:T], g[:, cut:T], beta[:, cut:T], h_a)
    assert torch.equal(o_a, o_all[:, :cut])
    _check('o (second call)', o_all[:, cut:].float().cpu(), o_b, 2e-3)
    _check('ht (chained)', h_all.cpu(), h_b, 1e-3)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    dev = 'cuda'
    o_d, h_d = fused_recurrent_gated_delta_rule(q[:, T:].to(dev), k[:, T:].to(dev), v[:, T:].to(dev), g[:, T:].to(dev),
                                                beta=beta[:, T:].to(dev), initial_state=h_all, output_final_state=True)
    _check('o (decode)', ref_o[:, T:], o_d)
    _check('ht (decode)', ref_ht, h_d)


def test_wide_keys_outputs_fully_written_and_deterministic():
    """Every element of o and ht is written (NaN-filled allocator pool) and two runs agree bit for bit."""
    B, T, H, HV, K, V = 2, 450, 2, 4, 256, 200
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, K, V, seed=21, gate_div=4.0, h0_std=0.5, dtype=torch.bfloat16)
    junk = [torch.full((1 << 22,), float('nan'), device='cuda') for _ in range(8)]
    del junk
    o1, h1 = _run(q, k, v, g, beta, h0)
    assert not torch.isnan(o1.float()).any() and not torch.isnan(h1).any()
    o2, h2 = _run(q, k, v, g, beta, h0)
    assert torch.equal(o1, o2) and torch.equal(h1, h2)


@pytest.mark.parametrize('case', ['fast', 'slow', 'mixed'])
def test_wide_keys_time_segments_that_start_warm(monkeypatch, case):
    """A long dense sequence on few heads is cut into time segments that start warm (a zero state a few chunks early, decided
    per head on the device from the bound on the chunks' transitions); a head that decays too slowly for that takes the exact
    start states of a first pass and a merge (fla/ops/common/intracard_cp.py:139-180 does the same inside one card), bit
    for bit what the run with exact start states forced for every head gives it."""
    B, T, H, HV, K, V = 1, 8192, 2, 4, 256, 256                # 16 workgroups per segment: 16 segments of 8 chunks in either mode
    q, k, v, _, beta, h0 = O.make_inputs(B, T, H, HV, K, V, seed=31, h0_std=0.5, dtype=torch.bfloat16)
    per_token = {'fast': [0.1] * 4, 'slow': [1e-3] * 4, 'mixed': [0.1, 1e-3, 0.3, 0.005]}[case]
    gen = torch.Generator().manual_seed(32)
    g = -(0.5 + torch.rand(B, T, HV, generator=gen)) * torch.tensor(per_token)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    o_s, h_s = _run(q, k, v, g, beta, h0)
    _check('o', ref_o, o_s)
    _check('ht', ref_ht, h_s)
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', 'segments-exact')
    o_e, h_e = _run(q, k, v, g, beta, h0)
    _check('o (exact start states)', ref_o, o_e)
    _check('ht (exact start states)', ref_ht, h_e)
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', 'wide')
    o_w, h_w = _run(q, k, v, g, beta, h0)
    slow_heads = {'fast': [], 'slow': [0, 1, 2, 3], 'mixed': [1, 3]}[case]
    for hv in range(HV):
        same = torch.equal(o_s[:, :, hv], o_e[:, :, hv]) and torch.equal(h_s[:, hv], h_e[:, hv])
        # (the first segment starts from the true state in every form)
        assert torch.equal(o_s[:, :512, hv], o_w[:, :512, hv]) and torch.equal(o_e[:, :512, hv], o_w[:, :512, hv]), hv
        if hv in slow_heads:
            assert same, f'head {hv} cannot start warm and must take the exact start states'
        else:
            assert not same, hv                                 # a different, equally good start
        # (two evaluations with 16-bit operands, each within the bar of the oracle)
        assert O.get_err_ratio(o_w[:, :, hv].float().cpu(), o_e[:, :, hv].float().cpu()) < 7e-3, hv


def test_wide_keys_exact_segments_layer_shape(monkeypatch):
    """The reference layer's default head shape (K = 256, V = 512) on a prompt long enough for time segments, with gates that
    hardly decay (no segment can start warm: first pass, merge of 256-row states, second pass), V-first states and a final state."""
    B, T, H, HV, K, V = 1, 8192, 2, 2, 256, 512                # 16 segments of 8 chunks in either mode
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, K, V, seed=41, gate_div=512.0, h0_std=0.5, dtype=torch.bfloat16)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    o, ht = _run(q, k, v, g, beta, h0.transpose(-1, -2).contiguous(), state_v_first=True)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht.transpose(-1, -2))
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', 'segments-exact')
    o_e, h_e = _run(q, k, v, g, beta, h0.transpose(-1, -2).contiguous(), state_v_first=True)
    assert torch.equal(o, o_e) and torch.equal(ht, h_e)           # the automatic choice took that path by itself
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', 'wide')
    o_w, h_w = _run(q, k, v, g, beta, h0.transpose(-1, -2).contiguous(), state_v_first=True)
    assert not torch.equal(o, o_w)
    _check('o (whole sequences)', ref_o, o_w)
    # K below 256 and value columns past the last block: rows and columns of the segment buffers that no run writes
    B, T, H, HV, K, V = 1, 2048, 1, 2, 192, 200
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, K, V, seed=42, gate_div=512.0, h0_std=0.5, dtype=torch.bfloat16)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    junk = [torch.full((1 << 22,), float('nan'), device='cuda') for _ in range(8)]
    del junk
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', 'segments-exact')
    o, ht = _run(q, k, v, g, beta, h0)
    _check('o (K = 192, V = 200)', ref_o, o)
    _check('ht (K = 192, V = 200)', ref_ht, ht)
