"""GPU parity of chunk_gated_delta_rule (HIP, through the C ABI) against the fp32 CPU oracle
on the same seeded inputs.  Cases follow the reference's matrix for this operator
(tests/ops/test_gdn.py:108-200, :712-878, :1350-1478; tests/ops/test_gdn_kernels.py:587-627)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu

# o and final state: relative RMSE <= 5e-3 and max-abs-error ratio <= 1e-2 vs the fp32 oracle
RATIO, MAXABS = 5e-3, 1e-2


def _op():
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    return chunk_gated_delta_rule


def _check(name, ref, got, ratio=RATIO, maxabs=MAXABS):
    got = got.detach().float().cpu()
    assert got.shape == ref.shape, f'{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}'
    assert not torch.isnan(got).any(), f'{name}: NaN'
    r, m = O.get_err_ratio(ref, got), O.max_abs_ratio(ref, got)
    assert r <= ratio and m <= maxabs, f'{name}: rel-rmse {r:.3e} max-abs ratio {m:.3e}'
    return r, m


def _run(q, k, v, g, beta, h0=None, cu=None, **kw):
    dev = 'cuda'
    cu_t = None if cu is None else torch.tensor(cu, dtype=kw.pop('idx_dtype', torch.int64), device=dev)
    return _op()(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta.to(dev),
                 initial_state=None if h0 is None else h0.to(dev), output_final_state=True, cu_seqlens=cu_t, **kw)


@pytest.mark.parametrize('B,T,H,HV,D,gate_div,with_h0,dtype', [
    (1, 64, 1, 1, 128, 1.0, False, torch.bfloat16),
    (2, 256, 2, 2, 128, 1.0, False, torch.bfloat16),
    (1, 130, 2, 4, 128, 16.0, True, torch.bfloat16),       # GVA, ragged tail chunk, non-zero h0
    (2, 1000, 2, 8, 128, 16.0, True, torch.bfloat16),
    (2, 75, 2, 2, 128, 1.0, True, torch.float16),
    (1, 1024, 4, 4, 128, 16.0, True, torch.float16),
    (2, 512, 2, 2, 64, 1.0, True, torch.bfloat16),         # padded to 128 on the host
    (2, 500, 2, 4, 60, 16.0, True, torch.float16),
    (1, 300, 3, 3, 100, 1.0, False, torch.bfloat16),
    (2, 256, 2, 2, 64, 1.0, False, torch.float32),         # config 1 shape; fp32 inputs run as bf16
])
def test_chunk_vs_oracle(B, T, H, HV, D, gate_div, with_h0, dtype):
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, D, D, seed=42, gate_div=gate_div,
                                         h0_std=0.5 if with_h0 else None, dtype=dtype)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    o, ht = _run(q, k, v, g, beta, h0)
    assert o.dtype == q.dtype and ht.dtype == torch.float32
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('B,T,H,HV,D,scale,gate_logit_normalizer,mask_p,l2norm_in_kernel', [
    (4, 1024, 4, 4, 128, 0.1, 1, 1.0, False),
    (2, 75, 4, 4, 64, 1, 0.01, 0, False),
    (2, 500, 3, 3, 60, 1, 1, 0, False),
    (2, 1000, 3, 3, 64, 0.1, 1, 0.5, False),
    (3, 1024, 4, 4, 100, 1, 0.1, 0, False),
    (4, 1024, 4, 4, 128, 0.1, 1, 0, True),
    (2, 1500, 4, 4, 128, 0.1, 10, 0, False),
    (4, 2048, 8, 8, 64, 0.1, 1, 0, False),
    (2, 256, 2, 4, 64, 1, 1, 0, False),
    (2, 512, 2, 8, 64, 1, 0.1, 0, True),
    (2, 1024, 4, 8, 128, 0.1, 1, 0, False),
])
def test_reference_matrix_with_the_reference_input_recipe(B, T, H, HV, D, scale, gate_logit_normalizer, mask_p, l2norm_in_kernel):
    """The reference's own parameter matrix and input recipe for this operator (tests/ops/test_gdn.py:108-200):
    fp16, q/k/v uniform in [0, 1) (strongly correlated keys), gates divided by the normaliser (0.01 = decay
    by e^-69 per token), a fraction mask_p of the gates set to zero, zero initial state, custom scale, l2
    normalisation outside or inside the kernels.  Its bar: error ratio 0.005 on o and ht."""
    gen = torch.Generator().manual_seed(42)
    dtype = torch.float16
    q = torch.rand(B, T, H, D, generator=gen).to(dtype)
    k = torch.rand(B, T, H, D, generator=gen).to(dtype)
    v = torch.rand(B, T, HV, D, generator=gen).to(dtype)
    beta = torch.rand(B, T, HV, generator=gen).sigmoid()
    g = F.logsigmoid(torch.rand(B, T, HV, generator=gen)) / gate_logit_normalizer
    g = g * (torch.rand(B, T, HV, generator=gen) > mask_p)
    h0 = torch.zeros(B, HV, D, D)
    qn, kn = F.normalize(q.float(), p=2, dim=-1).to(dtype), F.normalize(k.float(), p=2, dim=-1).to(dtype)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(qn, kn, v, g, beta, scale, h0, True)
    dev = 'cuda'
    o, ht = _op()((q if l2norm_in_kernel else qn).to(dev), (k if l2norm_in_kernel else kn).to(dev), v.to(dev), g.to(dev),
                  beta.to(dev), scale=scale, initial_state=h0.to(dev), output_final_state=True,
                  use_qk_l2norm_in_kernel=l2norm_in_kernel)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('H,HV,D,mask_p,cu', [
    (4, 4, 60, 0, [0, 15]),
    (4, 4, 64, 0, [0, 256, 500, 1000]),
    (4, 4, 64, 0.5, [0, 256, 500, 1000]),
    (4, 4, 100, 0, [0, 15, 100, 300, 1200, 2000]),
    (2, 4, 64, 0, [0, 256, 500, 1000]),
    (2, 8, 64, 0, [0, 256, 500, 1000]),
])
def test_reference_varlen_matrix_with_the_reference_input_recipe(H, HV, D, mask_p, cu):
    """The reference's packed-input matrix and recipe (tests/ops/test_gdn.py:712-800): fp16, q NOT
    normalised, k normalised, fp16 gates with a masked fraction, fp16 initial states of unit variance;
    every sequence is checked against the token recurrence run on it alone.  Bar 0.005."""
    gen = torch.Generator().manual_seed(42)
    dtype = torch.float16
    T, N = cu[-1], len(cu) - 1
    q = torch.randn(1, T, H, D, generator=gen).to(dtype)
    k = F.normalize(torch.randn(1, T, H, D, generator=gen), p=2, dim=-1).to(dtype)
    v = torch.randn(1, T, HV, D, generator=gen).to(dtype)
    g = F.logsigmoid(torch.rand(1, T, HV, generator=gen)).to(dtype)
    g = g * (torch.rand(1, T, HV, generator=gen) > mask_p)
    beta = torch.rand(1, T, HV, generator=gen).sigmoid()
    h0 = torch.randn(N, HV, D, D, generator=gen).to(dtype)
    refs = [O.recurrent_gated_delta_rule(q[:, a:b], k[:, a:b], v[:, a:b], g[:, a:b].float(), beta[:, a:b], None,
                                         h0[i:i + 1].float(), True) for i, (a, b) in enumerate(zip(cu[:-1], cu[1:]))]
    ref_o, ref_ht = torch.cat([r[0] for r in refs], 1), torch.cat([r[1] for r in refs], 0)
    o, ht = _run(q, k, v, g, beta, h0, cu)
    assert ht.dtype == torch.float32
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('B,T,H,HV,D,scale,has_dt_bias,l2norm_in_kernel', [
    (2, 75, 4, 4, 64, 1, True, True),
    (2, 500, 3, 3, 60, 1, False, False),
    (2, 1000, 3, 3, 64, 0.1, True, False),
    (3, 1024, 4, 4, 100, 1, True, True),
    (4, 1024, 4, 4, 128, 0.1, False, True),
    (4, 2048, 8, 8, 64, 0.1, True, False),
    (2, 256, 2, 4, 64, 1, True, False),             # grouped value heads (:1000-1104)
    (2, 512, 1, 4, 64, 0.1, False, False),
    (2, 512, 2, 8, 64, 1, True, False),
    (2, 1024, 4, 8, 128, 0.1, True, False),
])
def test_reference_gate_in_kernel_matrix_with_the_reference_input_recipe(B, T, H, HV, D, scale, has_dt_bias, l2norm_in_kernel):
    """tests/ops/test_gdn.py:878-1104: raw gate inputs ~ N(0,1), A_log ~ N(0,1) per value head (decays up to
    e^-20 and more per token), optional dt_bias, fp16 uniform q/k/v, zero initial state; the gate activation
    -exp(A_log)*softplus(g + dt_bias) happens inside the first kernel.  Bar 0.005."""
    gen = torch.Generator().manual_seed(42)
    dtype = torch.float16
    q = torch.rand(B, T, H, D, generator=gen).to(dtype)
    k = torch.rand(B, T, H, D, generator=gen).to(dtype)
    v = torch.rand(B, T, HV, D, generator=gen).to(dtype)
    beta = torch.rand(B, T, HV, generator=gen).sigmoid()
    g_raw = torch.randn(B, T, HV, generator=gen)
    A_log = torch.randn(HV, generator=gen)
    dt_bias = torch.randn(HV, generator=gen) if has_dt_bias else None
    h0 = torch.zeros(B, HV, D, D)
    qn, kn = F.normalize(q.float(), p=2, dim=-1).to(dtype), F.normalize(k.float(), p=2, dim=-1).to(dtype)
    g_ref = -A_log.exp() * F.softplus(g_raw + (dt_bias if has_dt_bias else 0.0))        # gate.py:21-46
    ref_o, ref_ht = O.recurrent_gated_delta_rule(qn, kn, v, g_ref, beta, scale, h0, True)
    dev = 'cuda'
    o, ht = _op()((q if l2norm_in_kernel else qn).to(dev), (k if l2norm_in_kernel else kn).to(dev), v.to(dev),
                  g_raw.to(dev), beta.to(dev), scale=scale, initial_state=h0.to(dev), output_final_state=True,
                  use_qk_l2norm_in_kernel=l2norm_in_kernel, use_gate_in_kernel=True, A_log=A_log.to(dev),
                  dt_bias=None if dt_bias is None else dt_bias.to(dev))
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('mode', ['auto', 'wide-single', 'wide-pair', 'segments-single', 'segments-exact-single', 'segments-pair'])
@pytest.mark.parametrize('B,T,H,HV,K,V,vfirst,cu', [
    (2, 1100, 2, 4, 64, 64, False, None),
    (1, 1300, 2, 2, 32, 96, True, None),
    (2, 900, 1, 2, 128, 64, False, None),
    (1, 2000, 2, 4, 64, 128, True, [0, 15, 100, 300, 1200, 2000]),
    (1, 777, 2, 4, 8, 8, False, None),
])
def test_head_dims_that_are_multiples_of_8_go_to_the_kernels_as_they_are(monkeypatch, mode, B, T, H, HV, K, V, vfirst, cu):
    """No padded copies on the host: the kernels read rows of K or V elements, keep key features past K at
    zero and never store value columns past V.  Guard rows and columns around the outputs stay untouched."""
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', mode)
    N = B if cu is None else len(cu) - 1
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, K, V, seed=17, gate_div=8.0, h0_std=0.5, N=N, dtype=torch.bfloat16)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu_seqlens=cu)
    from fla_hip.ops.gated_delta_rule.chunk import ChunkLaunch
    from fla_hip.ops.gated_delta_rule._common import ptr
    dev = 'cuda'
    hs = (h0.transpose(-1, -2) if vfirst else h0).contiguous().to(dev)
    cu_t = None if cu is None else torch.tensor(cu, device=dev)
    call = ChunkLaunch(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta.to(dev), K ** -0.5, hs, True, vfirst, cu_t)
    assert call.padded == (K, V)
    # the outputs sit inside larger buffers filled with a guard value
    o_big = torch.full((B * T * HV * V + 256,), 7.0, dtype=torch.bfloat16, device=dev)
    h_big = torch.full((N * HV * K * V + 256,), 7.0, dtype=torch.float32, device=dev)
    args = list(call.args)
    assert args[9] == ptr(call.o) and args[8] == ptr(call.ht)
    args[9], args[8] = o_big.data_ptr() + 128 * 2, h_big.data_ptr() + 128 * 4
    call.args = tuple(args)
    call.run()
    torch.cuda.synchronize()
    o = o_big[128:128 + B * T * HV * V].view(B, T, HV, V)
    ht = h_big[128:128 + N * HV * K * V].view((N, HV, V, K) if vfirst else (N, HV, K, V))
    assert torch.all(o_big[:128] == 7.0) and torch.all(o_big[-128:] == 7.0), 'output guard overwritten'
    assert torch.all(h_big[:128] == 7.0) and torch.all(h_big[-128:] == 7.0), 'state guard overwritten'
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht.transpose(-1, -2) if vfirst else ht)


@torch.inference_mode()
def test_reference_varlen_prefill_case_under_inference_mode():
    """tests/ops/test_gdn.py:806-876, its largest case: one packed sequence of 8192 tokens, D = 60, fp16
    everywhere (q unnormalised, gates, beta and initial state in fp16), called under inference mode."""
    gen = torch.Generator().manual_seed(42)
    dtype, H, D, cu = torch.float16, 4, 60, [0, 8192]
    T = cu[-1]
    q = torch.randn(1, T, H, D, generator=gen).to(dtype)
    k = F.normalize(torch.randn(1, T, H, D, generator=gen), p=2, dim=-1).to(dtype)
    v = torch.randn(1, T, H, D, generator=gen).to(dtype)
    g = F.logsigmoid(torch.rand(1, T, H, generator=gen)).to(dtype)
    beta = torch.rand(1, T, H, generator=gen).to(dtype).sigmoid()
    h0 = torch.randn(1, H, D, D, generator=gen).to(dtype)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g.float(), beta.float(), None, h0.float(), True)
    o, ht = _run(q, k, v, g, beta, h0, cu)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('mode', ['wide-single', 'segments-single', 'segments-exact-single', 'wide-pair', 'segments-pair'])
@pytest.mark.parametrize('B,T,H,HV,with_h0,vfirst', [
    (2, 1000, 2, 4, True, False),
    (1, 2100, 2, 2, True, True),          # ragged tail, V-first state layout
    (3, 512, 1, 2, False, False),
])
def test_every_form_of_the_sequential_stage(monkeypatch, mode, B, T, H, HV, with_h0, vfirst):
    """The forms of the sequential stage (one workgroup for the whole sequence or time segments
    with fp32 merge; two runs per workgroup or one) are interchangeable: each must meet the
    oracle on its own."""
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', mode)
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, 128, 128, seed=21, gate_div=16.0,
                                         h0_std=0.5 if with_h0 else None, dtype=torch.bfloat16)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    if vfirst:
        o, ht = _run(q, k, v, g, beta, h0.transpose(-1, -2).contiguous(), state_v_first=True)
        ht = ht.transpose(-1, -2)
    else:
        o, ht = _run(q, k, v, g, beta, h0)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


def _gates_per_head(B, T, HV, per_token, seed):
    """log-decays of size `per_token[hv]` (times a random factor in [0.5, 1.5]) per value head"""
    gen = torch.Generator().manual_seed(seed)
    return -(0.5 + torch.rand(B, T, HV, generator=gen)) * torch.tensor(per_token)


@pytest.mark.parametrize('case', ['fast', 'slow', 'mixed', 'expanding', 'boundary'])
def test_segments_that_start_warm(monkeypatch, case):
    """Time segments start from a zero state a few chunks early where the decay over those chunks makes
    the true state irrelevant (bound 2^-32), and from the exact merged state otherwise - decided per head
    on the device.  Heads that decay slowly, or whose keys are long enough to stretch the state
    (beta |k|^2 > 2), must take the exact path and then equal it bit for bit."""
    B, T, H, HV, D = 1, 8192, 4, 16, 128          # 16 segments of 8 chunks; up to 16 chunks of warm-up
    q, k, v, _, beta, h0 = O.make_inputs(B, T, H, HV, D, D, seed=31, h0_std=0.5, dtype=torch.bfloat16)
    per_token = {'fast': [0.05] * 16, 'slow': [1e-4] * 16, 'mixed': [0.05, 1e-4, 0.2, 0.01] * 4,
                 'expanding': [0.05] * 16, 'boundary': [0.0875] * 16}[case]
    g = _gates_per_head(B, T, HV, per_token, seed=32)
    if case == 'expanding':
        k = (k.float() * 1.6).bfloat16()          # beta |k|^2 up to 2.56: some tokens stretch the state
        beta = torch.ones_like(beta)
        g = g * 4                                   # (keeps the recurrence itself stable)
    if case == 'boundary':
        # constant decay: 8.08 in log2 units per chunk, so 4 chunks give 2^-32.3 and 3 do not: the warm-up length is exactly 4
        g = torch.full_like(g, -0.0875)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    out = {}
    for mode in ('segments-single', 'segments-exact-single'):
        monkeypatch.setenv('FLA_HIP_SCAN_MODE', mode)
        out[mode] = _run(q, k, v, g, beta, h0)
        _check(f'o {mode}', ref_o, out[mode][0])
        _check(f'ht {mode}', ref_ht, out[mode][1])
    (o_w, h_w), (o_e, h_e) = out['segments-single'], out['segments-exact-single']
    same = torch.equal(o_w, o_e) and torch.equal(h_w, h_e)
    if case in ('slow', 'expanding'):
        assert same, 'heads that cannot start warm must take the exact path unchanged'
    else:
        # a different (and equally good) start state: close; with a decay that varies it is not identical
        # (with the constant decay of 'boundary' what a warm start drops may lie below the rounding of the fp32 state)
        assert case == 'boundary' or not same
        # (bf16 rounding of the operands: two EXACT evaluations - whole sequences and segments from merged states - differ
        # by 2.1e-3 from each other on these inputs, each 3.7e-3 from the fp32 oracle)
        assert O.get_err_ratio(o_e.float().cpu(), o_w.float().cpu()) < 3e-3
    if case == 'mixed':
        # per head: value heads 1 and 3 decay too slowly (1e-4, 0.01 per token) and are bitwise those of the exact path
        assert torch.equal(o_w[:, :, 1::2], o_e[:, :, 1::2]) and torch.equal(h_w[:, 1::2], h_e[:, 1::2])
        # (heads 2, 6, ... decay so fast that a warm start reproduces the exact fp32 state: nothing to tell apart)
        for hv in range(0, 16, 4):
            assert not torch.equal(o_w[:, :, hv], o_e[:, :, hv]), hv


def test_warm_start_forgets_an_enormous_state(monkeypatch):
    """What a warm start drops is bounded by 2^-32 of the state BEFORE the warm-up chunks: an initial state and early
    values a million times the size of what follows (1e6 x 2^-32 = 2e-4, below the operator's bar) must leave the later
    output as accurate as the exact path."""
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', 'segments-single')
    B, T, H, HV, D = 1, 8192, 4, 16, 128
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, D, D, seed=33, gate_div=4.0, h0_std=1e6, dtype=torch.bfloat16)
    v = v.float()
    v[:, :512] *= 1e6
    v = v.bfloat16()
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, dtype=torch.float64)
    o, ht = _run(q, k, v, g, beta, h0)
    _check('ht', ref_ht.float(), ht)
    _check('o (late tokens)', ref_o[:, 4096:].float(), o[:, 4096:])


@pytest.mark.parametrize('mode', ['wide-pair', 'segments-pair'])
@pytest.mark.parametrize('B,T,H,HV,dtype,gate_div', [
    (1, 1991, 1, 4, torch.float16, 16.0),       # f16 (state rescaled every chunk), four value heads per q/k head, ragged tail
    (2, 1300, 3, 6, torch.bfloat16, 1.0),       # strong decay: the lazy rescaling of the state fires
    (1, 4160, 2, 2, torch.bfloat16, 16.0),      # one value head per q/k head: only pass 1 can pair its runs
])
def test_two_runs_per_workgroup(monkeypatch, mode, B, T, H, HV, dtype, gate_div):
    """Shapes that stress what only the two-run kernel has: its own copies and counted waits over many
    chunks, the masked output stores of a partial last chunk, teams with different value heads or with
    the S / M runs of one head, and the idle team of the first segment."""
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', mode)
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, 128, 128, seed=5, gate_div=gate_div, h0_std=0.5, dtype=dtype)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    o, ht = _run(q, k, v, g, beta, h0)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    # rows past the end of a sequence are never written: guard rows behind the output keep their value
    if B == 1:
        from fla_hip.ops.gated_delta_rule.chunk import ChunkLaunch
        from fla_hip.ops.gated_delta_rule._common import ptr
        dev = 'cuda'
        Tm = T - 13
        a = [x[:, :Tm].to(dev).contiguous() for x in (q, k, v, g, beta)]
        call = ChunkLaunch(*a, 128 ** -0.5, h0.to(dev), True)
        big = torch.full((1, Tm + 64, HV, 128), 7.0, dtype=dtype, device=dev)
        args = list(call.args)
        assert args[9] == ptr(call.o)
        args[9] = ptr(big)
        call.args = tuple(args)
        call.run()
        torch.cuda.synchronize()
        assert torch.all(big[:, Tm:] == 7.0), 'tokens past the end of the sequence were written'
        ref_m = O.chunk_gated_delta_rule(q[:, :Tm], k[:, :Tm], v[:, :Tm], g[:, :Tm], beta[:, :Tm], None, h0, True)[0]
        _check('o (shorter call)', ref_m, big[:, :Tm])


@pytest.mark.parametrize('B,T,H,HV,K,V,vfirst,cu', [
    (2, 300, 2, 2, 128, 256, False, None),      # wide values: split into two 128-column heads
    (1, 500, 2, 4, 64, 200, True, None),        # ... padded, V-first state layout
    (1, 700, 1, 2, 100, 384, False, [0, 130, 131, 700]),
    (2, 150, 2, 2, 256, 128, False, None),      # wide keys: the scan kernel with 64 value columns per workgroup
    (1, 200, 1, 2, 192, 192, True, [0, 77, 200]),
])
def test_head_dims_above_128(B, T, H, HV, K, V, vfirst, cu):
    """Every shape the reference accepts (K <= 256, any V: fla/ops/common/chunk_delta_h.py:712) gives the right answer
    through the chunk entry point."""
    N = B if cu is None else len(cu) - 1
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, K, V, seed=31, gate_div=8.0, h0_std=0.5, N=N, dtype=torch.bfloat16)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu_seqlens=cu)
    if vfirst:
        o, ht = _run(q, k, v, g, beta, h0.transpose(-1, -2).contiguous(), cu, state_v_first=True)
        ht = ht.transpose(-1, -2)
    else:
        o, ht = _run(q, k, v, g, beta, h0, cu)
    assert o.shape == (B, T, HV, V) and o.dtype == q.dtype
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


def test_key_dim_above_256_is_rejected():
    q, k, v, g, beta, _ = O.make_inputs(1, 64, 1, 1, 320, 64, seed=1, dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        _run(q, k, v, g, beta)


@pytest.mark.parametrize('mode', ['auto', 'single', 'pair'])
def test_varlen_every_form(monkeypatch, mode):
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', mode)
    cu = [0, 1, 100, 101, 300, 1200, 2000]
    q, k, v, g, beta, h0 = O.make_inputs(1, cu[-1], 2, 4, 128, 128, seed=23, gate_div=2.0, h0_std=0.5, N=6, dtype=torch.float16)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu_seqlens=cu)
    o, ht = _run(q, k, v, g, beta, h0, cu)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


def test_against_token_recurrence_and_decode_handoff():
    """Prefill with the chunk op, continue with the recurrent op: equals one long recurrence."""
    from fla_hip.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    q, k, v, g, beta, h0 = O.make_inputs(2, 300, 2, 4, 128, 128, seed=7, gate_div=4.0, h0_std=0.3, dtype=torch.bfloat16)
    ref_o, ref_ht = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    dev = 'cuda'
    a = [x.to(dev) for x in (q, k, v, g, beta)]
    o1, h1 = _op()(*(x[:, :290] for x in a), initial_state=h0.to(dev), output_final_state=True)
    o2, h2 = fused_recurrent_gated_delta_rule(a[0][:, 290:], a[1][:, 290:], a[2][:, 290:], a[3][:, 290:], beta=a[4][:, 290:],
                                              initial_state=h1, output_final_state=True)
    _check('o', ref_o, torch.cat([o1, o2], 1))
    _check('ht', ref_ht, h2)


@pytest.mark.parametrize('cu,H,HV,D', [
    ([0, 15], 2, 2, 128),
    ([0, 256, 500, 1000], 2, 4, 128),
    ([0, 1, 100, 101, 300, 1200, 2000], 2, 8, 128),
    ([0, 15, 100, 300, 1200, 2000], 2, 4, 64),
])
@pytest.mark.parametrize('idx_dtype', [torch.int64, torch.int32])
@pytest.mark.parametrize('mode', ['wide-single', 'wide-pair'])
def test_varlen_vs_oracle_and_bit_exact_ownership(monkeypatch, cu, H, HV, D, idx_dtype, mode):
    # the form of the sequential kernel is pinned so that the packed call and the single-sequence
    # calls run the very same code: any difference is then a token or state given to the wrong sequence
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', mode)
    T, N = cu[-1], len(cu) - 1
    q, k, v, g, beta, h0 = O.make_inputs(1, T, H, HV, D, D, seed=11, gate_div=2.0, h0_std=0.5, N=N, dtype=torch.bfloat16)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu_seqlens=cu)
    o, ht = _run(q, k, v, g, beta, h0, cu, idx_dtype=idx_dtype)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    # every sequence run alone through the same kernels reproduces the packed result bit for bit
    for n, (s, e) in enumerate(zip(cu[:-1], cu[1:])):
        o_n, h_n = _run(q[:, s:e], k[:, s:e], v[:, s:e], g[:, s:e], beta[:, s:e], h0[n:n + 1])
        assert torch.equal(o_n[0], o[0, s:e]), f'sequence {n}: o differs'
        assert torch.equal(h_n[0], ht[n]), f'sequence {n}: state differs'


def test_many_documents_equals_two_halves():
    """More (document, head) pairs than a 16-bit grid dimension holds
    (tests/ops/test_gdn_kernels.py:587-627): 2050 documents of 16 tokens, HV = 32."""
    ND, L, H, D = 2050, 16, 32, 128
    T = ND * L
    gen = torch.Generator().manual_seed(0)
    q = F.normalize(torch.randn(1, T, H, D, generator=gen), dim=-1).bfloat16()
    k = F.normalize(torch.randn(1, T, H, D, generator=gen), dim=-1).bfloat16()
    v = torch.randn(1, T, H, D, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(1, T, H, generator=gen))
    beta = torch.sigmoid(torch.randn(1, T, H, generator=gen))
    cu = list(range(0, T + 1, L))
    o, ht = _run(q, k, v, g, beta, None, cu)
    half = (ND // 2) * L
    o1, h1 = _run(q[:, :half], k[:, :half], v[:, :half], g[:, :half], beta[:, :half], None, cu[:ND // 2 + 1])
    o2, h2 = _run(q[:, half:], k[:, half:], v[:, half:], g[:, half:], beta[:, half:], None,
                  [c - half for c in cu[ND // 2:]])
    assert torch.equal(torch.cat([o1, o2], 1), o) and torch.equal(torch.cat([h1, h2], 0), ht)
    # spot-check a few documents against the oracle
    for n in (0, 1024, 2049):
        s, e = cu[n], cu[n + 1]
        ref_o, ref_h = O.recurrent_gated_delta_rule(q[:, s:e], k[:, s:e], v[:, s:e], g[:, s:e], beta[:, s:e], None, None, True)
        _check(f'o[{n}]', ref_o[0], o[0, s:e])
        _check(f'ht[{n}]', ref_h[0], ht[n])


def test_flags_and_state_layout():
    B, T, H, HV, D = 2, 200, 2, 4, 128
    gen = torch.Generator().manual_seed(5)
    q, k = torch.randn(B, T, H, D, generator=gen).bfloat16(), torch.randn(B, T, H, D, generator=gen).bfloat16()
    v = torch.randn(B, T, HV, D, generator=gen).bfloat16()
    graw, braw = torch.randn(B, T, HV, generator=gen), torch.randn(B, T, HV, generator=gen)
    A_log, dt_bias = 0.3 * torch.randn(HV, generator=gen), 0.3 * torch.randn(HV, generator=gen)
    h0 = 0.5 * torch.randn(B, HV, D, D, generator=gen)
    kw = dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True, use_beta_sigmoid_in_kernel=True, allow_neg_eigval=False)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, graw, braw, None, h0, True, A_log=A_log, dt_bias=dt_bias, **kw)
    o, ht = _run(q, k, v, graw, braw, h0, A_log=A_log.cuda(), dt_bias=dt_bias.cuda(), **kw)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    o2, ht2 = _run(q, k, v, graw, braw, h0.transpose(-1, -2).contiguous(), A_log=A_log.cuda(), dt_bias=dt_bias.cuda(),
                   state_v_first=True, **kw)
    assert ht2.shape == (B, HV, D, D)
    assert torch.equal(o2, o) and torch.equal(ht2.transpose(-1, -2), ht)      # same kernels, transposed I/O only
    for cs in (16, 32):
        o3, ht3 = _run(q, k, v, graw, braw, h0, A_log=A_log.cuda(), dt_bias=dt_bias.cuda(), chunk_size=cs, **kw)
        _check(f'o chunk_size={cs}', ref_o, o3)


@pytest.mark.parametrize('kw', [
    dict(use_qk_l2norm_in_kernel=True),
    dict(use_gate_in_kernel=True),
    dict(use_gate_in_kernel=True, dt_bias=None),
    dict(use_beta_sigmoid_in_kernel=True),
    dict(use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True),
    dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True, use_beta_sigmoid_in_kernel=True, allow_neg_eigval=True),
])
def test_each_prologue_inside_the_kernels_packed_input(kw):
    """l2 normalisation of q and k, gate activation and beta sigmoid are applied by the kernels
    (as row factors / on the fly); each alone and all together must meet the oracle, here on packed
    sequences with grouped value heads and ragged tails."""
    cu = [0, 70, 71, 400, 1000]
    T, N, H, HV, D = cu[-1], len(cu) - 1, 2, 4, 128
    gen = torch.Generator().manual_seed(17)
    q, k = 3 * torch.randn(1, T, H, D, generator=gen).bfloat16(), 0.3 * torch.randn(1, T, H, D, generator=gen).bfloat16()
    if not kw.get('use_qk_l2norm_in_kernel'):
        q, k = F.normalize(q.float(), dim=-1).bfloat16(), F.normalize(k.float(), dim=-1).bfloat16()
    v = torch.randn(1, T, HV, D, generator=gen).bfloat16()
    g = torch.randn(1, T, HV, generator=gen)
    if not kw.get('use_gate_in_kernel'):
        g = F.logsigmoid(g) / 4
    beta = torch.randn(1, T, HV, generator=gen)
    if not kw.get('use_beta_sigmoid_in_kernel'):
        beta = torch.sigmoid(beta)
    h0 = 0.5 * torch.randn(N, HV, D, D, generator=gen)
    kw = dict(kw)
    ref_kw, run_kw = dict(kw), dict(kw)
    if kw.get('use_gate_in_kernel'):
        A_log = 0.3 * torch.randn(HV, generator=gen)
        dt_bias = None if 'dt_bias' in kw else 0.3 * torch.randn(HV, generator=gen)
        ref_kw.update(A_log=A_log, dt_bias=dt_bias)
        run_kw.update(A_log=A_log.cuda(), dt_bias=None if dt_bias is None else dt_bias.cuda())
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True, cu_seqlens=cu, **ref_kw)
    o, ht = _run(q, k, v, g, beta, h0, cu, **run_kw)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('mode,T', [('auto', 333), ('wide-single', 2100), ('wide-pair', 2100), ('segments-single', 4200), ('segments-exact-single', 4200), ('segments-pair', 4200)])
def test_outputs_fully_written_and_deterministic(monkeypatch, mode, T):
    """Two runs agree bit for bit and every output element is written (no NaN survives from
    poisoned allocations: the workspace and outputs come from torch.empty).  Every form of the
    sequential stage: a copy that is awaited too early or too late shows up as a difference
    between runs sooner than as an error against the oracle."""
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', mode)
    q, k, v, g, beta, h0 = O.make_inputs(2, T, 2, 4, 128, 128, seed=3, gate_div=8.0, h0_std=0.2, dtype=torch.bfloat16)
    junk = torch.full((64, 1024, 1024), float('nan'), device='cuda')      # poison the caching allocator's pool
    del junk
    o1, h1 = _run(q, k, v, g, beta, h0)
    for _ in range(3):
        junk = torch.full((64, 1024, 1024), float('nan'), device='cuda')
        del junk
        o2, h2 = _run(q, k, v, g, beta, h0)
        assert torch.equal(o1, o2) and torch.equal(h1, h2)
    assert not torch.isnan(o1).any() and not torch.isnan(h1).any()


def test_host_validation_errors():
    op = _op()
    dev = 'cuda'
    q = torch.randn(2, 64, 2, 128, device=dev, dtype=torch.bfloat16)
    v = torch.randn(2, 64, 4, 128, device=dev, dtype=torch.bfloat16)
    g = torch.zeros(2, 64, 4, device=dev)
    with pytest.raises(ValueError):
        op(q, q[:, :, :1], v, g, g)                                              # q/k head mismatch
    with pytest.raises(ValueError):
        op(q, q, v[:, :, :3], g[:, :, :3], g[:, :, :3])                          # HV % H
    with pytest.raises(ValueError):
        op(q, q, v, g, g, chunk_size=48)
    with pytest.raises(ValueError):
        op(q, q, v, g, g, cu_seqlens=torch.tensor([0, 64, 128], device=dev))     # batch must be 1
    with pytest.raises(ValueError):
        op(q[:1], q[:1], v[:1], g[:1], g[:1], initial_state=torch.zeros(3, 4, 128, 128, device=dev),
           cu_seqlens=torch.tensor([0, 32, 64], device=dev))
    with pytest.raises(ValueError):
        op(q, q, v, g, g, allow_neg_eigval=True)
    with pytest.raises(AssertionError):
        op(q, q, v, g, g, use_gate_in_kernel=True)
    with pytest.raises(DeprecationWarning):
        op(q, q, v, g, g, head_first=True)
    with pytest.raises(RuntimeError):
        op(q.cpu(), q.cpu(), v.cpu(), g.cpu(), g.cpu())                          # no CPU path


@pytest.mark.parametrize('B,T,H,HV,D,dtype', [
    (1, 1024, 4, 4, 128, torch.bfloat16),
    (2, 2048, 8, 8, 128, torch.bfloat16),
    (1, 4096, 16, 16, 128, torch.bfloat16),
    (1, 1024, 4, 4, 128, torch.float16),
    (2, 2048, 8, 8, 128, torch.float16),
    (1, 1024, 2, 8, 128, torch.bfloat16),           # grouped value heads
    (2, 2048, 4, 16, 128, torch.bfloat16),
])
def test_reference_whole_operator_backend_matrix(B, T, H, HV, D, dtype):
    """The matrix and recipe with which the reference checks a whole-operator backend (its closest analogue of this
    library; tests/ops/test_gdn.py:1350-1403): everything `randn`, unit-variance fp32 initial states, l2 norm in
    the kernel, scale D^-0.5, against the token recurrence on normalised q, k.  The reference's bar is 0.008."""
    gen = torch.Generator().manual_seed(42)
    q = torch.randn(B, T, H, D, generator=gen).to(dtype)
    k = torch.randn(B, T, H, D, generator=gen).to(dtype)
    v = torch.randn(B, T, HV, D, generator=gen).to(dtype)
    g = F.logsigmoid(torch.randn(B, T, HV, generator=gen))
    beta = torch.randn(B, T, HV, generator=gen).sigmoid()
    h0 = torch.randn(B, HV, D, D, generator=gen)
    ref_o, ref_ht = O.chunk_gated_delta_rule(O.l2norm(q.float()), O.l2norm(k.float()), v, g, beta, D ** -0.5, h0, True)
    o, ht = _run(q, k, v, g, beta, h0, scale=D ** -0.5, use_qk_l2norm_in_kernel=True)
    _check('o', ref_o, o, ratio=0.008)
    _check('ht', ref_ht, ht, ratio=0.008)


@pytest.mark.parametrize('H,D,cu', [
    (4, 128, [0, 256, 500, 1000]),
    (8, 128, [0, 100, 300, 1200, 2000]),
    (16, 128, [0, 101, 303, 1205, 3007, 4096]),
])
def test_reference_whole_operator_backend_matrix_packed(H, D, cu):
    """The packed-input half of the same check (tests/ops/test_gdn.py:1406-1478): bf16, every sequence against the
    token recurrence run on it alone."""
    gen = torch.Generator().manual_seed(42)
    dtype, T, N = torch.bfloat16, cu[-1], len(cu) - 1
    q = torch.randn(1, T, H, D, generator=gen).to(dtype)
    k = torch.randn(1, T, H, D, generator=gen).to(dtype)
    v = torch.randn(1, T, H, D, generator=gen).to(dtype)
    g = F.logsigmoid(torch.randn(1, T, H, generator=gen))
    beta = torch.randn(1, T, H, generator=gen).sigmoid()
    h0 = torch.randn(N, H, D, D, generator=gen)
    refs = [O.recurrent_gated_delta_rule(O.l2norm(q[:, a:b].float()), O.l2norm(k[:, a:b].float()), v[:, a:b], g[:, a:b],
                                         beta[:, a:b], D ** -0.5, h0[i:i + 1], True) for i, (a, b) in enumerate(zip(cu[:-1], cu[1:]))]
    ref_o, ref_ht = torch.cat([r[0] for r in refs], 1), torch.cat([r[1] for r in refs], 0)
    o, ht = _run(q, k, v, g, beta, h0, cu, scale=D ** -0.5, use_qk_l2norm_in_kernel=True)
    _check('o', ref_o, o, ratio=0.008)
    _check('ht', ref_ht, ht, ratio=0.008)
