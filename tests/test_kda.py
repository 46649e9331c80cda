"""The KDA operator's token recurrence (fused_recurrent_kda, fused_recurrent_kda_fwd: a decay per key feature) on the
gated delta rule's HIP recurrence kernel, through gdn_fused_recurrent_kda_fwd, against the CPU oracle.  Shapes, input
recipes and the 0.005 bar of the reference's own tests (tests/ops/test_kda.py:100-330: fp32, q and k uniform in [0, 1)
and normalised, g = logsigmoid(randn) / normalizer, beta = sigmoid(randn), random initial state)."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu
RATIO = 5e-3


def _ops():
    from fla_hip.ops.kda import fused_recurrent_kda, fused_recurrent_kda_fwd
    return fused_recurrent_kda, fused_recurrent_kda_fwd


def _check(name, ref, got, ratio=RATIO):
    got = got.detach().float().cpu()
    assert got.shape == ref.shape, f'{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}'
    assert not torch.isnan(got).any(), f'{name}: NaN'
    r, m = O.get_err_ratio(ref, got), O.max_abs_ratio(ref, got)
    assert r <= ratio and m <= 1e-2, f'{name}: rel-rmse {r:.3e} max-abs ratio {m:.3e}'


def _inputs(B, T, H, HV, D, dtype=torch.float32, normalizer=1.0, seed=42, raw_gate=False):
    gen = torch.Generator().manual_seed(seed)
    q = torch.rand(B, T, H, D, generator=gen).to(dtype)
    k = torch.rand(B, T, H, D, generator=gen).to(dtype)
    v = torch.rand(B, T, HV, D, generator=gen).to(dtype)
    g = torch.randn(B, T, HV, D, generator=gen)
    if not raw_gate:
        g = F.logsigmoid(g) / normalizer
    beta = torch.randn(B, T, HV, generator=gen).to(dtype).sigmoid()
    h0 = torch.randn(B, HV, D, D, generator=gen)
    return q, k, v, g, beta, h0


def _cuda(*xs):
    return [None if x is None else x.cuda() for x in xs]


@pytest.mark.parametrize('B,T,H,HV,D,scale,normalizer,l2,dtype', [
    (1, 64, 1, 1, 64, 1, 1, False, torch.float32),
    (2, 512, 3, 3, 60, 1, 1, False, torch.float32),
    (3, 1000, 4, 4, 100, 0.1, 1, True, torch.float32),
    (4, 1024, 4, 4, 128, 0.1, 1, False, torch.float32),
    (2, 512, 2, 4, 60, 1, 1, False, torch.float32),
    (2, 1024, 2, 8, 128, 0.1, 1, True, torch.float32),
    (2, 300, 2, 4, 128, 0.1, 10, True, torch.bfloat16),
    (1, 200, 2, 2, 256, 1, 1, False, torch.float16),
])
def test_fused_recurrent_kda_reference_matrix(B, T, H, HV, D, scale, normalizer, l2, dtype):
    q, k, v, g, beta, h0 = _inputs(B, T, H, HV, D, dtype, normalizer)
    if not l2:
        q, k = F.normalize(q.float(), p=2, dim=-1).to(dtype), F.normalize(k.float(), p=2, dim=-1).to(dtype)
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, scale, h0, True, use_qk_l2norm_in_kernel=l2)
    dq, dk, dv, dg, db, dh = _cuda(q, k, v, g, beta, h0)
    keep = dh.clone()
    o, ht = _ops()[0](dq, dk, dv, dg, db, scale=scale, initial_state=dh, output_final_state=True, use_qk_l2norm_in_kernel=l2)
    assert o.dtype == dtype and ht.dtype == torch.float32 and torch.equal(dh, keep)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)


@pytest.mark.parametrize('B,T,H,D,neg', [(2, 256, 4, 64, False), (2, 256, 4, 64, True), (1, 512, 3, 60, True)])
def test_fused_recurrent_kda_beta_sigmoid_in_kernel(B, T, H, D, neg):
    q, k, v, g, beta_post, h0 = _inputs(B, T, H, H, D)
    q, k = F.normalize(q, p=2, dim=-1), F.normalize(k, p=2, dim=-1)
    beta_raw = torch.logit(beta_post.clamp(1e-4, 1 - 1e-4))
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta_post * (2 if neg else 1), None, h0, True)
    dq, dk, dv, dg, db, dh = _cuda(q, k, v, g, beta_raw, h0)
    o, ht = _ops()[0](dq, dk, dv, dg, db, initial_state=dh, output_final_state=True,
                      use_beta_sigmoid_in_kernel=True, allow_neg_eigval=neg)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    with pytest.raises(ValueError, match='allow_neg_eigval'):
        _ops()[0](dq, dk, dv, dg, db, allow_neg_eigval=True)


@pytest.mark.parametrize('B,T,H,D,scale', [(1, 64, 1, 64, 1), (2, 512, 3, 60, 1), (3, 1000, 4, 100, 0.1), (4, 1024, 4, 128, 0.1)])
def test_fused_recurrent_kda_state_v_first(B, T, H, D, scale):
    q, k, v, g, beta, h0 = _inputs(B, T, H, H, D)
    q, k = F.normalize(q, p=2, dim=-1), F.normalize(k, p=2, dim=-1)
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, scale, h0, True)
    dq, dk, dv, dg, db, dh = _cuda(q, k, v, g, beta, h0.transpose(-1, -2).contiguous())
    o, ht = _ops()[0](dq, dk, dv, dg, db, scale=scale, initial_state=dh, output_final_state=True, state_v_first=True)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht.transpose(-1, -2))


@pytest.mark.parametrize('mode', ['softplus', 'softplus-no-bias', 'bounded', 'bounded-no-A', 'softplus-no-A'])
@pytest.mark.parametrize('H,HV,D,vfirst', [(2, 4, 64, False), (3, 3, 100, True), (2, 2, 128, False)])
def test_fused_recurrent_kda_gate_in_kernel(mode, H, HV, D, vfirst):
    """The raw gate activated in the kernel (fla/ops/kda/fused_recurrent.py:168-181): both forms, with and without
    A_log and the bias [HV * K]; the reference's layer draws A_log = log(U(1, 16)) and a bias of softplus-inverse values."""
    B, T = 2, 150
    q, k, v, g, beta, h0 = _inputs(B, T, H, HV, D, raw_gate=True, seed=7)
    gen = torch.Generator().manual_seed(8)
    A_log = torch.log(1 + 15 * torch.rand(HV, generator=gen)) if 'no-A' not in mode else None
    dt_bias = torch.randn(HV * D, generator=gen) if 'no-bias' not in mode else None
    lower = -5.0 if mode.startswith('bounded') else None
    if mode == 'softplus':
        g = g - 4.0                      # (keeps the decay of 150 tokens from wiping the state)
    kw = dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True, lower_bound=lower)
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, None, h0, True, A_log=A_log, dt_bias=dt_bias, **kw)
    kw['state_v_first'] = vfirst
    dq, dk, dv, dg, db, dh, dA, dbias = _cuda(q, k, v, g, beta, h0.transpose(-1, -2).contiguous() if vfirst else h0, A_log, dt_bias)
    o, ht = _ops()[0](dq, dk, dv, dg, db, A_log=dA, dt_bias=dbias, initial_state=dh, output_final_state=True, **kw)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht.transpose(-1, -2) if vfirst else ht)
    # the gate applied on the host and passed as log decays gives the same numbers up to the activation's rounding
    gk = O.kda_gate(g, A_log, dt_bias, lower).cuda()
    o2, ht2 = _ops()[0](dq, dk, dv, gk, db, initial_state=dh, output_final_state=True, use_qk_l2norm_in_kernel=True, state_v_first=vfirst)
    _check('o (host gate)', o2.float().cpu(), o, 1e-4)
    _check('ht (host gate)', ht2.cpu(), ht, 1e-4)


@pytest.mark.parametrize('mode', ['log-decay', 'softplus', 'bounded-no-A'])
@pytest.mark.parametrize('T,dtype', [(1, torch.bfloat16), (3, torch.float32)])
def test_fused_recurrent_kda_decode_kernel(mode, T, dtype):
    """1024 states of K = V = 128 and more take the whole-state decode kernels in their form with a decay per key feature:
    both state layouts against the oracle and against the general kernel (the same sequences in two calls of 512 states)."""
    B, H, HV, D = 128, 4, 8, 128
    q, k, v, g, beta, h0 = _inputs(B, T, H, HV, D, dtype=dtype, raw_gate=mode != 'log-decay', seed=11)
    gen = torch.Generator().manual_seed(12)
    A_log = torch.log(1 + 15 * torch.rand(HV, generator=gen)) if mode == 'softplus' else None
    dt_bias = torch.randn(HV * D, generator=gen) if mode != 'log-decay' else None
    lower = -5.0 if mode.startswith('bounded') else None
    if mode == 'softplus':
        g = g - 4.0
    kw = dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=mode != 'log-decay', lower_bound=lower)
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, None, h0, True, A_log=A_log, dt_bias=dt_bias, **kw)
    dq, dk, dv, dg, db, dh, dA, dbias = _cuda(q, k, v, g, beta, h0, A_log, dt_bias)
    o, ht = _ops()[0](dq, dk, dv, dg, db, A_log=dA, dt_bias=dbias, initial_state=dh, output_final_state=True, **kw)
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    o2, ht2 = _ops()[0](dq, dk, dv, dg, db, A_log=dA, dt_bias=dbias, initial_state=dh.transpose(-1, -2).contiguous(),
                        output_final_state=True, state_v_first=True, **kw)
    _check('o (V-first decode kernel)', o2.float().cpu(), o, 1e-4)
    _check('ht (V-first decode kernel)', ht2.transpose(-1, -2).cpu(), ht, 1e-4)
    # (512 states at a time go to the general kernel)
    halves = [_ops()[0](dq[a:b], dk[a:b], dv[a:b], dg[a:b], db[a:b], A_log=dA, dt_bias=dbias, initial_state=dh[a:b],
                        output_final_state=True, **kw) for a, b in ((0, 64), (64, 128))]
    _check('o (general kernel)', torch.cat([x[0] for x in halves]).float().cpu(), o, 1e-4)
    _check('ht (general kernel)', torch.cat([x[1] for x in halves]).cpu(), ht, 1e-4)
    # the serving form: states updated in place
    from fla_hip.ops.kda import fused_recurrent_kda_fwd
    pool = dh.clone()
    o3, _ = fused_recurrent_kda_fwd(dq, dk, dv, dg, db, A_log=dA, dt_bias=dbias, initial_state=pool, inplace_final_state=True, **kw)
    assert torch.equal(o3, o) and torch.equal(pool, ht)


@pytest.mark.parametrize('idx_dtype', [torch.int64, torch.int32])
def test_fused_recurrent_kda_packed(idx_dtype):
    cu = [0, 15, 16, 100, 356, 357, 1000]
    T, N, H, HV, D = cu[-1], len(cu) - 1, 2, 4, 64
    q, k, v, g, beta, _ = _inputs(1, T, H, HV, D, seed=3)
    h0 = torch.randn(N, HV, D, D, generator=torch.Generator().manual_seed(4))
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, None, h0, True, cu_seqlens=cu, use_qk_l2norm_in_kernel=True)
    dq, dk, dv, dg, db, dh = _cuda(q, k, v, g, beta, h0)
    o, ht = _ops()[0](dq, dk, dv, dg, db, initial_state=dh, output_final_state=True, use_qk_l2norm_in_kernel=True,
                      cu_seqlens=torch.tensor(cu, dtype=idx_dtype, device='cuda'))
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    with pytest.raises(ValueError, match='number of initial states'):
        _ops()[0](dq, dk, dv, dg, db, initial_state=dh[:2], cu_seqlens=torch.tensor(cu, device='cuda'))
    with pytest.raises(ValueError, match='batch size is expected to be 1'):
        _ops()[0](dq.expand(2, -1, -1, -1), dk, dv, dg, db, cu_seqlens=torch.tensor(cu, device='cuda'))


def test_fused_recurrent_kda_fwd_state_pool_and_speculative_decoding():
    """The serving form (fla/ops/kda/fused_recurrent.py:236-338): states in a pool, in place by default; a slot per
    sequence, and a slot per token with the start taken from the slot of the last accepted token."""
    N, H, HV, D, slots = 5, 2, 4, 64, 23
    fwd = _ops()[1]
    gen = torch.Generator().manual_seed(11)
    pool = torch.randn(slots, HV, D, D, generator=gen)
    # one token per sequence, a slot per sequence, gate activated in the kernel
    q, k, v, g, beta, _ = _inputs(N, 1, H, HV, D, raw_gate=True, seed=12)
    A_log, dt_bias = torch.log(1 + 15 * torch.rand(HV, generator=gen)), torch.randn(HV * D, generator=gen)
    idx = torch.randperm(slots, generator=gen)[:N]
    kw = dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=True)
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, None, pool[idx], True, A_log=A_log, dt_bias=dt_bias, **kw)
    dq, dk, dv, dg, db, dpool, dA, dbias = _cuda(q, k, v, g, beta, pool, A_log, dt_bias)
    o, ret = fwd(dq, dk, dv, dg, db, A_log=dA, dt_bias=dbias, initial_state=dpool, ssm_state_indices=idx.cuda(), **kw)
    assert ret.data_ptr() == dpool.data_ptr()
    _check('o', ref_o, o)
    _check('pool slots', ref_ht, dpool[idx.cuda()])
    rest = [i for i in range(slots) if i not in idx.tolist()]
    assert torch.equal(dpool[rest].cpu(), pool[rest])
    # three draft tokens per sequence, a slot per token, starts from the slot of the last accepted token
    T = 3
    q, k, v, g, beta, _ = _inputs(N, T, H, HV, D, seed=13)
    idx2 = torch.randperm(slots, generator=gen)[:N * T].view(N, T).to(torch.int32)
    acc = torch.tensor([1, 3, 2, 1, 2], dtype=torch.int32)
    gk = g
    ref_o, ref_pool, _ = O.recurrent_gated_delta_rule_pooled(q, k, v, None, beta, D ** -0.5, pool, idx2, acc, gk=gk, use_qk_l2norm_in_kernel=True)
    dq, dk, dv, dg, db, dpool = _cuda(q, k, v, g, beta, pool)
    o, _ = fwd(dq, dk, dv, dg, db, initial_state=dpool, ssm_state_indices=idx2.cuda(), num_accepted_tokens=acc.cuda(),
               use_qk_l2norm_in_kernel=True)
    _check('o (speculative)', ref_o, o)
    _check('pool (speculative)', ref_pool, dpool)
    # `out` receives the result; in-place without a state is refused
    buf = torch.empty_like(dv)
    o2, _ = fwd(dq, dk, dv, dg, db, initial_state=dpool.clone(), ssm_state_indices=idx2.cuda(), num_accepted_tokens=acc.cuda(),
                use_qk_l2norm_in_kernel=True, out=buf)
    assert o2.data_ptr() == buf.data_ptr()
    with pytest.raises(ValueError, match='requires `initial_state`'):
        fwd(dq, dk, dv, dg, db)


def test_kda_entry_point_argument_checks():
    from fla_hip import _lib
    lib = _lib.load()
    x = torch.zeros(2, 1, 2, 64, device='cuda')
    g = torch.zeros(2, 1, 2, 64, device='cuda')
    b = torch.zeros(2, 1, 2, device='cuda')
    A = torch.zeros(2, device='cuda')
    args = lambda A_log, mode, flags: (x.data_ptr(), x.data_ptr(), x.data_ptr(), g.data_ptr(), b.data_ptr(), A_log, None, 0.0, mode,
                                        None, None, x.data_ptr(), None, None, None, 1, 2, 1, 2, 2, 64, 64, 2, 1.0,
                                        _lib.DTYPE_F32, _lib.DTYPE_F32, flags, None)
    assert lib.gdn_fused_recurrent_kda_fwd(*args(None, 3, 0)) == _lib.GDN_ERR_INVALID and 'gate_mode' in _lib.last_error()
    assert lib.gdn_fused_recurrent_kda_fwd(*args(A.data_ptr(), 0, 0)) == _lib.GDN_ERR_INVALID and 'A_log' in _lib.last_error()
    assert lib.gdn_fused_recurrent_kda_fwd(*args(None, 0, _lib.FLAG_STATE_BF16)) == _lib.GDN_ERR_UNSUPPORTED
    assert lib.gdn_fused_recurrent_kda_fwd(*args(A.data_ptr(), 1, 0)) == _lib.GDN_OK
    torch.cuda.synchronize()


def test_upstream_kda_backend_takes_gpu_inference_calls_and_leaves_the_rest():
    """The backend for upstream's 'kda' registry (fla/ops/kda/backends/__init__.py:14), through this package's mirror of
    the registry: GPU inference calls of fused_recurrent_kda_fwd run the HIP kernel, everything else the default."""
    from fla_hip.ops.backends import BackendRegistry, BaseBackend, dispatch
    from fla_hip.upstream import make_kda_backend
    BackendRegistry('upstream_test_kda').register(make_kda_backend(BaseBackend)())

    @dispatch('upstream_test_kda')
    def fused_recurrent_kda_fwd(q, k, v, g, beta, A_log=None, dt_bias=None, initial_state=None, scale=None,
                                output_final_state=False, inplace_final_state=True, **kwargs):
        return 'default', None

    q, k, v, g, beta, h0 = _inputs(2, 5, 2, 4, 64)
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, None, h0, True, use_qk_l2norm_in_kernel=True)
    dq, dk, dv, dg, db, dh = _cuda(q, k, v, g, beta, h0)
    o, ht = fused_recurrent_kda_fwd(dq, dk, dv, dg, db, initial_state=dh, use_qk_l2norm_in_kernel=True)
    assert ht.data_ptr() == dh.data_ptr()                    # in place by default, as upstream
    _check('o', ref_o, o)
    _check('ht', ref_ht, ht)
    assert fused_recurrent_kda_fwd(q, k, v, g, beta, initial_state=h0)[0] == 'default'                       # CPU stays upstream
    assert fused_recurrent_kda_fwd(dq.requires_grad_(), dk, dv, dg, db, initial_state=dh)[0] == 'default'    # training stays upstream
    assert fused_recurrent_kda_fwd(dq.detach(), dk, dv, dg, db, initial_state=dh.bfloat16())[0] == 'default'

    @dispatch('upstream_test_kda')
    def chunk_kda(q, k, v, g, beta, scale=None, initial_state=None, output_final_state=False, **kwargs):
        return 'default', None

    q, k, v, g, beta, h0 = _inputs(1, 150, 2, 4, 64)
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, None, h0, True, use_qk_l2norm_in_kernel=True)
    dq, dk, dv, dg, db, dh = _cuda(q, k, v, g, beta, h0)
    o, ht = chunk_kda(dq.bfloat16(), dk.bfloat16(), dv.bfloat16(), dg, db, initial_state=dh, output_final_state=True,
                      use_qk_l2norm_in_kernel=True)
    assert O.get_err_ratio(ref_o, o.float().cpu()) < 0.01 and O.get_err_ratio(ref_ht, ht.cpu()) < 0.01
    assert chunk_kda(q, k, v, g, beta)[0] == 'default'                                                        # CPU stays upstream
    qg = dq.bfloat16().requires_grad_()
    o2, _ = chunk_kda(qg, dk.bfloat16(), dv.bfloat16(), dg, db, initial_state=dh, use_qk_l2norm_in_kernel=True)      # training calls too
    o2.float().square().sum().backward()
    assert torch.equal(o2, o) and qg.grad is not None and bool(qg.grad.float().abs().sum() > 0)
    wide = torch.zeros(1, 150, 2, 192, device='cuda', dtype=torch.bfloat16)
    assert chunk_kda(wide, wide, dv.bfloat16(), torch.zeros(1, 150, 4, 192, device='cuda'), db)[0] == 'default'


# --------------------------------------------------------------------------------------------
# chunked prefill (chunk_kda) against the oracle's token recurrence
# --------------------------------------------------------------------------------------------
def _chunk_inputs(B, T, H, HV, D, gate_div, mask_p, gate_in_kernel, safe_gate, dtype, seed=42, V=None):
    gen = torch.Generator().manual_seed(seed)
    V = D if V is None else V
    q = torch.rand(B, T, H, D, generator=gen).to(dtype)
    k = torch.rand(B, T, H, D, generator=gen).to(dtype)
    v = torch.rand(B, T, HV, V, generator=gen).to(dtype)
    g = torch.randn(B, T, HV, D, generator=gen)
    A_log = dt_bias = None
    if gate_in_kernel:
        A_log = torch.randn(HV, generator=gen)
        dt_bias = torch.randn(HV * D, generator=gen)
    else:
        g = F.logsigmoid(g) / gate_div
        g = g * (torch.rand(B, T, HV, D, generator=gen) > mask_p)
        if safe_gate:
            g = g.clamp(-5, 0)
    beta = torch.randn(B, T, HV, generator=gen).sigmoid()
    h0 = torch.randn(B, HV, D, V, generator=gen)
    return q, k, v, g, beta, h0, A_log, dt_bias


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,HV,D,scale,gate_div,mask_p,l2,gate_in_kernel,dtype,safe_gate', [
    (1, 63, 1, 1, 64, 1, 1, 0, False, False, torch.float16, True),          # the reference's matrix, tests/ops/test_kda.py:535-560
    (2, 500, 3, 3, 60, 1, 1, 0, False, False, torch.float16, True),
    (2, 1000, 3, 3, 64, 0.1, 1, 0.5, False, False, torch.float16, False),
    (3, 1024, 4, 4, 100, 1, 0.1, 0, False, False, torch.float16, False),
    (4, 1024, 4, 4, 128, 0.1, 1, 0, False, False, torch.float16, True),
    (4, 1024, 4, 4, 128, 0.1, 1, 0, True, False, torch.float16, True),
    (2, 1500, 4, 4, 128, 0.1, 10, 0, False, True, torch.float16, False),
    (4, 2048, 8, 8, 64, 0.1, 1, 0, False, True, torch.float16, True),
    (2, 1024, 2, 4, 64, 0.1, 1, 0, False, False, torch.float16, False),
    (2, 1024, 2, 8, 64, 0.1, 1, 0, False, True, torch.float16, False),
    (2, 1024, 4, 8, 128, 0.1, 1, 0, True, True, torch.float16, False),
    (2, 1024, 2, 4, 64, 0.1, 1, 0, True, True, torch.bfloat16, True),
    (2, 1024, 2, 8, 128, 0.1, 1, 0, True, True, torch.bfloat16, False),
])
def test_chunk_kda_reference_matrix(B, T, H, HV, D, scale, gate_div, mask_p, l2, gate_in_kernel, dtype, safe_gate):
    from fla_hip.ops.kda import chunk_kda
    q, k, v, g, beta, h0, A_log, dt_bias = _chunk_inputs(B, T, H, HV, D, gate_div, mask_p, gate_in_kernel, safe_gate, dtype)
    lower_bound = -5.0 if safe_gate else None
    if not l2:
        q, k = F.normalize(q.float(), p=2, dim=-1).to(dtype), F.normalize(k.float(), p=2, dim=-1).to(dtype)
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, scale, h0, True, use_qk_l2norm_in_kernel=l2,
                                    use_gate_in_kernel=gate_in_kernel, A_log=A_log, dt_bias=dt_bias, lower_bound=lower_bound)
    dev = 'cuda'
    d = lambda x: None if x is None else x.to(dev)
    o, ht = chunk_kda(d(q), d(k), d(v), d(g), d(beta), scale=scale, initial_state=d(h0), output_final_state=True,
                      use_qk_l2norm_in_kernel=l2, use_gate_in_kernel=gate_in_kernel, A_log=d(A_log), dt_bias=d(dt_bias),
                      safe_gate=safe_gate, lower_bound=lower_bound)
    assert o.dtype == dtype and ht.dtype == torch.float32 and o.shape == v.shape
    # (the reference's bars for o and the final state: tests/ops/test_kda.py:640-641)
    assert O.get_err_ratio(ref_o, o.float().cpu()) < 0.005
    assert O.get_err_ratio(ref_ht, ht.cpu()) < 0.005


@pytest.mark.gpu
@pytest.mark.parametrize('H,D,mask_p,cu,gate_in_kernel,safe_gate', [
    (4, 60, 0.1, [0, 15], True, False),
    (4, 64, 0.9, [0, 256, 500, 1000], True, False),
    (4, 128, 0.5, [0, 256, 500, 1000], False, False),
    (4, 100, 0, [0, 15, 100, 300, 1200, 2000], True, False),
    (2, 128, 0, [0, 1, 65, 65, 200], False, True),
])
def test_chunk_kda_packed(H, D, mask_p, cu, gate_in_kernel, safe_gate):
    """Packed sequences (tests/ops/test_kda.py:839-960), one of them empty, int32 boundaries, every sequence alone = packed."""
    from fla_hip.ops.kda import chunk_kda
    T, N = cu[-1], len(cu) - 1
    dtype = torch.float16
    q, k, v, g, beta, _, A_log, dt_bias = _chunk_inputs(1, T, H, H, D, 1.0, mask_p, gate_in_kernel, safe_gate, dtype, seed=7)
    gen = torch.Generator().manual_seed(8)
    h0 = torch.randn(N, H, D, D, generator=gen)
    lower_bound = -5.0 if safe_gate else None
    kw = dict(use_qk_l2norm_in_kernel=True, use_gate_in_kernel=gate_in_kernel, lower_bound=lower_bound)
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, None, h0, True, cu_seqlens=cu, A_log=A_log, dt_bias=dt_bias, **kw)
    dev = 'cuda'
    d = lambda x: None if x is None else x.to(dev)
    cu_t = torch.tensor(cu, dtype=torch.int32, device=dev)
    o, ht = chunk_kda(d(q), d(k), d(v), d(g), d(beta), initial_state=d(h0), output_final_state=True, cu_seqlens=cu_t,
                      A_log=d(A_log), dt_bias=d(dt_bias), safe_gate=safe_gate, **kw)
    assert O.get_err_ratio(ref_o, o.float().cpu()) < 0.005 and O.get_err_ratio(ref_ht, ht.cpu()) < 0.005
    for n in range(N):
        s, e = cu[n], cu[n + 1]
        if e == s:
            assert torch.equal(ht[n].cpu(), h0[n])
            continue
        o1, ht1 = chunk_kda(d(q[:, s:e]), d(k[:, s:e]), d(v[:, s:e]), d(g[:, s:e]), d(beta[:, s:e]), initial_state=d(h0[n:n + 1]),
                            output_final_state=True, A_log=d(A_log), dt_bias=d(dt_bias), safe_gate=safe_gate, **kw)
        assert torch.equal(o1[0], o[0, s:e]) and torch.equal(ht1[0], ht[n])


@pytest.mark.gpu
@pytest.mark.parametrize('what', ['v_first', 'beta_sigmoid', 'beta_sigmoid_neg', 'wide_v', 'no_h0', 'strong_decay', 'bf16_hand_over'])
def test_chunk_kda_options(what):
    from fla_hip.ops.kda import chunk_kda, fused_recurrent_kda
    B, T, H, HV, D = 2, 200, 2, 4, 128
    V = 256 if what == 'wide_v' else D
    dtype = torch.bfloat16
    q, k, v, g, beta, h0, _, _ = _chunk_inputs(B, T, H, HV, D, 0.05 if what == 'strong_decay' else 4.0, 0, False, False, dtype, seed=3, V=V)
    kw = dict(use_qk_l2norm_in_kernel=True)
    gen = torch.Generator().manual_seed(4)
    if what.startswith('beta_sigmoid'):
        beta = torch.randn(B, T, HV, generator=gen)
        kw.update(use_beta_sigmoid_in_kernel=True, allow_neg_eigval=what.endswith('neg'))
    if what == 'no_h0':
        h0 = None
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, None, h0, True, **kw)
    dev = 'cuda'
    d = lambda x: None if x is None else x.to(dev)
    if what == 'v_first':
        o, ht = chunk_kda(d(q), d(k), d(v), d(g), d(beta), initial_state=d(h0.transpose(-1, -2).contiguous()), output_final_state=True,
                          state_v_first=True, **kw)
        ht = ht.transpose(-1, -2)
    else:
        o, ht = chunk_kda(d(q), d(k), d(v), d(g), d(beta), initial_state=d(h0), output_final_state=True, **kw)
    assert O.get_err_ratio(ref_o, o.float().cpu()) < 0.005 and O.get_err_ratio(ref_ht, ht.cpu()) < 0.005
    if what == 'bf16_hand_over':
        # prefill in two calls chained through the state, then a token of the recurrence: the same as one pass of the oracle
        o1, h1 = chunk_kda(d(q[:, :130]), d(k[:, :130]), d(v[:, :130]), d(g[:, :130]), d(beta[:, :130]), initial_state=d(h0),
                           output_final_state=True, **kw)
        o2, h2 = chunk_kda(d(q[:, 130:199]), d(k[:, 130:199]), d(v[:, 130:199]), d(g[:, 130:199]), d(beta[:, 130:199]),
                           initial_state=h1, output_final_state=True, **kw)
        o3, h3 = fused_recurrent_kda(d(q[:, 199:]), d(k[:, 199:]), d(v[:, 199:]), d(g[:, 199:]), d(beta[:, 199:]), initial_state=h2,
                                     output_final_state=True, **kw)
        joined = torch.cat([o1, o2, o3], dim=1)
        assert O.get_err_ratio(ref_o, joined.float().cpu()) < 0.005 and O.get_err_ratio(ref_ht, h3.cpu()) < 0.005


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,HV,D,V,l2,gate_in_kernel,safe_gate,vfirst,packed,dtype', [
    (2, 200, 2, 2, 256, 64, False, False, False, False, False, torch.bfloat16),
    (1, 300, 2, 4, 192, 128, True, True, False, True, False, torch.float16),
    (1, 260, 1, 2, 160, 200, False, True, True, False, True, torch.bfloat16),
])
def test_chunk_kda_wide_keys_forward(B, T, H, HV, D, V, l2, gate_in_kernel, safe_gate, vfirst, packed, dtype):
    """Key head dims above 128 (the reference allows up to 256, fla/ops/kda/chunk.py:409): forward only, on the token kernel."""
    from fla_hip.ops.kda import chunk_kda
    q, k, v, g, beta, h0, A_log, dt_bias = _chunk_inputs(B, T, H, HV, D, 1, 0, gate_in_kernel, safe_gate, dtype, V=V)
    lower_bound = -5.0 if safe_gate else None
    if not l2:
        q, k = F.normalize(q.float(), p=2, dim=-1).to(dtype), F.normalize(k.float(), p=2, dim=-1).to(dtype)
    cu = [0, 70, 71, T] if packed else None
    if packed:
        h0 = torch.randn(3, HV, D, V, generator=torch.Generator().manual_seed(7))
    if packed:
        outs = [O.recurrent_kda(q[:, a:b], k[:, a:b], v[:, a:b], g[:, a:b], beta[:, a:b], 0.1, h0[i:i + 1], True,
                                use_qk_l2norm_in_kernel=l2, use_gate_in_kernel=gate_in_kernel, A_log=A_log, dt_bias=dt_bias,
                                lower_bound=lower_bound) for i, (a, b) in enumerate(zip(cu[:-1], cu[1:]))]
        ref_o, ref_ht = torch.cat([x[0] for x in outs], 1), torch.cat([x[1] for x in outs], 0)
    else:
        ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, 0.1, h0, True, use_qk_l2norm_in_kernel=l2, use_gate_in_kernel=gate_in_kernel,
                                        A_log=A_log, dt_bias=dt_bias, lower_bound=lower_bound)
    d = lambda x: None if x is None else x.cuda()
    h0_in = h0.transpose(-1, -2).contiguous() if vfirst else h0
    o, ht = chunk_kda(d(q), d(k), d(v), d(g), d(beta), scale=0.1, initial_state=d(h0_in), output_final_state=True,
                      use_qk_l2norm_in_kernel=l2, use_gate_in_kernel=gate_in_kernel, A_log=d(A_log), dt_bias=d(dt_bias),
                      safe_gate=safe_gate, lower_bound=lower_bound, state_v_first=vfirst,
                      cu_seqlens=None if cu is None else torch.tensor(cu, device='cuda'))
    assert o.dtype == dtype and ht.dtype == torch.float32 and o.shape == v.shape
    ht = ht.transpose(-1, -2) if vfirst else ht
    assert O.get_err_ratio(ref_o, o.float().cpu()) < 0.005
    assert O.get_err_ratio(ref_ht, ht.cpu()) < 0.005
    # what this width does not have says so
    with pytest.raises(NotImplementedError, match='forward only'):
        chunk_kda(d(q).requires_grad_(True), d(k), d(v), d(g), d(beta), scale=0.1)
    with torch.inference_mode():
        with pytest.raises(NotImplementedError, match='intermediate'):
            chunk_kda(d(q), d(k), d(v), d(g), d(beta), scale=0.1, return_intermediate_states=True,
                      cu_seqlens=None if cu is None else torch.tensor(cu, device='cuda'))


@pytest.mark.gpu
def test_chunk_kda_validation():
    from fla_hip.ops.kda import chunk_kda
    x = torch.zeros(1, 64, 2, 64, dtype=torch.bfloat16, device='cuda')
    g = torch.zeros(1, 64, 2, 64, device='cuda')
    b = torch.zeros(1, 64, 2, device='cuda')
    with pytest.raises(ValueError):
        chunk_kda(x, x, x, g, b, allow_neg_eigval=True)
    with pytest.raises(ValueError):
        chunk_kda(x, x, x, g, b, safe_gate=True)
    with pytest.raises(ValueError):
        chunk_kda(x, x, x, g[..., :32], b)
    with pytest.raises(AssertionError, match='inference mode'):
        chunk_kda(x, x, x, g, b, return_intermediate_states=True)
    o, ht = chunk_kda(x[:, :0].detach(), x[:, :0].detach(), x[:, :0].detach(), g[:, :0], b[:, :0], output_final_state=True)
    assert o.shape == (1, 0, 2, 64) and torch.count_nonzero(ht) == 0


@pytest.mark.gpu
@pytest.mark.parametrize('seed', range(16))
def test_chunk_kda_random(seed):
    """Seeded random combinations of head dims, grouping, packing, gate form and range, prologues, state layout and dtype."""
    import random
    from fla_hip.ops.kda import chunk_kda
    rnd = random.Random(500 + seed)
    D = rnd.choice([16, 40, 64, 96, 128])
    V = rnd.choice([D, 64, 192]) if seed % 4 == 0 else D
    H = rnd.choice([1, 2, 3])
    HV = H * rnd.choice([1, 1, 2, 4])
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    if rnd.random() < 0.4:
        cu = [0]
        for _ in range(rnd.randint(1, 4)):
            cu.append(cu[-1] + rnd.choice([1, 7, 63, 64, 65, 130, 200]))
        B, T, N = 1, cu[-1], len(cu) - 1
    else:
        B, T, cu = rnd.randint(1, 3), rnd.choice([1, 5, 64, 100, 129, 257]), None
        N = B
    gen = torch.Generator().manual_seed(600 + seed)
    q, k = torch.randn(B, T, H, D, generator=gen).to(dtype), torch.randn(B, T, H, D, generator=gen).to(dtype)
    v = torch.randn(B, T, HV, V, generator=gen).to(dtype)
    kw = dict(use_qk_l2norm_in_kernel=True)
    A_log = dt_bias = None
    mode = rnd.choice(['plain', 'strong', 'softplus', 'lower_bound'])
    g = torch.randn(B, T, HV, D, generator=gen)
    if mode in ('plain', 'strong'):
        g = F.logsigmoid(g) / (0.05 if mode == 'strong' else rnd.choice([1.0, 8.0]))
    else:
        A_log = torch.randn(HV, generator=gen) * 0.5
        dt_bias = torch.randn(HV * D, generator=gen) * 0.5 if rnd.random() < 0.6 else None
        kw.update(use_gate_in_kernel=True)
        if mode == 'lower_bound':
            kw.update(lower_bound=-5.0, safe_gate=True)
    beta = torch.rand(B, T, HV, generator=gen).sigmoid()
    if rnd.random() < 0.3:
        beta = torch.randn(B, T, HV, generator=gen)
        kw.update(use_beta_sigmoid_in_kernel=True, allow_neg_eigval=rnd.random() < 0.5)
    h0 = torch.randn(N, HV, D, V, generator=gen) * 0.5 if rnd.random() < 0.7 else None
    okw = {n: x for n, x in kw.items() if n != 'safe_gate'}
    ref_o, ref_ht = O.recurrent_kda(q, k, v, g, beta, None, h0, True, cu_seqlens=cu, A_log=A_log, dt_bias=dt_bias, **okw)
    d = lambda x: None if x is None else x.cuda()
    vfirst = h0 is not None and rnd.random() < 0.3
    h_in = h0.transpose(-1, -2).contiguous() if vfirst else h0
    o, ht = chunk_kda(d(q), d(k), d(v), d(g), d(beta), initial_state=d(h_in), output_final_state=True, state_v_first=vfirst,
                      cu_seqlens=None if cu is None else torch.tensor(cu, device='cuda'), A_log=d(A_log), dt_bias=d(dt_bias), **kw)
    if vfirst:
        ht = ht.transpose(-1, -2)
    bar = 0.005 if T >= 64 else 0.01
    assert O.get_err_ratio(ref_o, o.float().cpu()) < bar and O.get_err_ratio(ref_ht, ht.cpu()) < bar


# --------------------------------------------------------------------------------------------
# backward of chunk_kda (gdn_chunk_kda_bwd) against the oracle's gradients
# --------------------------------------------------------------------------------------------
# (tests/ops/test_kda.py:651-661 of the reference; its 0.003 for dA only warns there, :659: held to 0.01 here)
GRAD_TOL = dict(dq=0.008, dk=0.008, dv=0.008, dg=0.02, dbeta=0.02, dh0=0.008, dA_log=0.01, ddt_bias=0.008)


def _kda_grads_gpu(q, k, v, g, beta, h0, A_log, dt_bias, do, dht, cu=None, **kw):
    from fla_hip.ops.kda import chunk_kda
    leaves = {n: (None if x is None else x.cuda().requires_grad_(True))
              for n, x in dict(dq=q, dk=k, dv=v, dg=g, dbeta=beta, dh0=h0, dA_log=A_log, ddt_bias=dt_bias).items()}
    cu_t = None if cu is None else torch.tensor(cu, dtype=kw.pop('idx_dtype', torch.int64), device='cuda')
    o, ht = chunk_kda(leaves['dq'], leaves['dk'], leaves['dv'], leaves['dg'], leaves['dbeta'], initial_state=leaves['dh0'],
                      output_final_state=True, A_log=leaves['dA_log'], dt_bias=leaves['ddt_bias'], cu_seqlens=cu_t, **kw)
    ((o.float() * do.cuda().float()).sum() + (ht * dht.cuda()).sum()).backward()
    return o, ht, {n: (None if x is None else x.grad) for n, x in leaves.items()}


def _compare_grads(ref, got, tol=GRAD_TOL):
    for n, r in ref.items():
        if r is None:
            continue
        x = got[n].detach().float().cpu()
        assert x.shape == r.shape, f'{n}: shape {tuple(x.shape)} vs {tuple(r.shape)}'
        assert not torch.isnan(x).any(), f'{n}: NaN'
        if O.get_abs_err(r, x) <= 1e-6:            # (fla/utils/_testing.py:28-34: gradients that vanish)
            continue
        e = O.get_err_ratio(r, x)
        assert e <= tol[n], f'{n}: rel-rmse {e:.3e} > {tol[n]}'


@pytest.mark.gpu
@pytest.mark.parametrize('B,T,H,HV,D,scale,gate_div,mask_p,l2,gate_in_kernel,dtype,safe_gate', [
    (1, 63, 1, 1, 64, 1, 1, 0, False, False, torch.float16, True),          # the reference's matrix (shorter where it is long)
    (2, 500, 3, 3, 60, 1, 1, 0, False, False, torch.float16, True),
    (2, 300, 3, 3, 64, 0.1, 1, 0.5, False, False, torch.float16, False),
    (2, 256, 4, 4, 100, 1, 0.1, 0, False, False, torch.float16, False),
    (2, 256, 4, 4, 128, 0.1, 1, 0, False, False, torch.float16, True),
    (2, 256, 4, 4, 128, 0.1, 1, 0, True, False, torch.float16, True),
    (2, 300, 4, 4, 128, 0.1, 10, 0, False, True, torch.float16, False),
    (2, 256, 8, 8, 64, 0.1, 1, 0, False, True, torch.float16, True),
    (2, 256, 2, 4, 64, 0.1, 1, 0, False, False, torch.float16, False),
    (2, 256, 2, 8, 64, 0.1, 1, 0, False, True, torch.float16, False),
    (2, 256, 4, 8, 128, 0.1, 1, 0, True, True, torch.float16, False),
    (2, 256, 2, 4, 64, 0.1, 1, 0, True, True, torch.bfloat16, True),
    (2, 256, 2, 4, 64, 0.1, 1, 0, False, True, torch.bfloat16, False),
    (2, 256, 2, 8, 128, 0.1, 1, 0, True, True, torch.bfloat16, False),
    (3, 100, 12, 24, 128, 0.1, 4.0, 0, False, False, torch.bfloat16, False),     # 72 runs: the scans take 64 value columns per workgroup
    (2, 70, 80, 80, 128, 0.1, 4.0, 0, False, False, torch.bfloat16, False),      # 160 runs: all 128
])
def test_chunk_kda_backward(B, T, H, HV, D, scale, gate_div, mask_p, l2, gate_in_kernel, dtype, safe_gate):
    q, k, v, g, beta, h0, A_log, dt_bias = _chunk_inputs(B, T, H, HV, D, gate_div, mask_p, gate_in_kernel, safe_gate, dtype)
    lower_bound = -5.0 if safe_gate else None
    if not l2:
        q, k = F.normalize(q.float(), p=2, dim=-1).to(dtype), F.normalize(k.float(), p=2, dim=-1).to(dtype)
    if gate_in_kernel:
        g = g.to(dtype)
    gen = torch.Generator().manual_seed(43)
    do = torch.randn(B, T, HV, D, generator=gen).to(dtype)
    dht = torch.randn(B, HV, D, D, generator=gen)
    kw = dict(scale=scale, use_qk_l2norm_in_kernel=l2, use_gate_in_kernel=gate_in_kernel, lower_bound=lower_bound)
    ref = O.kda_grads(q, k, v, g, beta, do, dht, initial_state=h0, A_log=A_log, dt_bias=dt_bias, dtype=torch.float32, **kw)
    o, ht, got = _kda_grads_gpu(q, k, v, g, beta, h0, A_log, dt_bias, do, dht, safe_gate=safe_gate, **kw)
    _compare_grads(ref, got)
    for n, x in dict(dq=q, dk=k, dv=v, dg=g, dbeta=beta, dh0=h0, dA_log=A_log, ddt_bias=dt_bias).items():
        if x is not None:
            assert got[n].dtype == x.dtype and got[n].shape == x.shape, n


@pytest.mark.gpu
@pytest.mark.parametrize('H,D,mask_p,cu,gate_in_kernel,safe_gate,idx_dtype', [
    (4, 60, 0.1, [0, 15], True, False, torch.int32),
    (4, 64, 0.9, [0, 256, 500, 1000], True, False, torch.int64),
    (4, 128, 0.5, [0, 256, 500, 1000], False, False, torch.int32),
    (4, 100, 0, [0, 15, 100, 300, 1200, 2000], True, False, torch.int64),
    (2, 128, 0, [0, 1, 65, 65, 200], False, True, torch.int64),
])
def test_chunk_kda_backward_packed(H, D, mask_p, cu, gate_in_kernel, safe_gate, idx_dtype):
    T, N = cu[-1], len(cu) - 1
    q, k, v, g, beta, _, A_log, dt_bias = _chunk_inputs(1, T, H, H, D, 1.0, mask_p, gate_in_kernel, safe_gate, torch.bfloat16)
    q, k = F.normalize(q.float(), p=2, dim=-1).bfloat16(), F.normalize(k.float(), p=2, dim=-1).bfloat16()
    lower_bound = -5.0 if safe_gate else None
    gen = torch.Generator().manual_seed(44)
    h0 = torch.randn(N, H, D, D, generator=gen)
    do = torch.randn(1, T, H, D, generator=gen).bfloat16()
    dht = torch.rand(N, H, D, D, generator=gen)
    kw = dict(use_gate_in_kernel=gate_in_kernel, lower_bound=lower_bound)
    ref = O.kda_grads(q, k, v, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, A_log=A_log, dt_bias=dt_bias, dtype=torch.float32, **kw)
    _, _, got = _kda_grads_gpu(q, k, v, g, beta, h0, A_log, dt_bias, do, dht, cu=cu, idx_dtype=idx_dtype, safe_gate=safe_gate, **kw)
    _compare_grads(ref, got)


@pytest.mark.gpu
@pytest.mark.parametrize('what', ['v_first', 'beta_sigmoid', 'beta_sigmoid_neg', 'wide_v', 'no_h0', 'strong_decay', 'outside_tokens'])
def test_chunk_kda_backward_options(what):
    B, T, H, HV, D = 2, 200, 2, 4, 64
    V = 200 if what == 'wide_v' else D
    q, k, v, g, beta, h0, _, _ = _chunk_inputs(B, T, H, HV, D, 0.02 if what == 'strong_decay' else 1.0, 0, False, False, torch.bfloat16, seed=5, V=V)
    q, k = F.normalize(q.float(), p=2, dim=-1).bfloat16(), F.normalize(k.float(), p=2, dim=-1).bfloat16()
    gen = torch.Generator().manual_seed(45)
    do = torch.randn(B, T, HV, V, generator=gen).bfloat16()
    kw, cu = {}, None
    if what == 'v_first':
        h0 = h0.transpose(-1, -2).contiguous()
        kw = dict(state_v_first=True)
    if what.startswith('beta_sigmoid'):
        beta = torch.randn(B, T, HV, generator=gen)
        kw = dict(use_beta_sigmoid_in_kernel=True, allow_neg_eigval=what.endswith('neg'))
    if what == 'no_h0':
        h0 = None
    dht = torch.randn(B, HV, V, D, generator=gen) if what == 'v_first' else torch.randn(B, HV, D, V, generator=gen)
    if what == 'outside_tokens':
        # a packed tensor whose sequences leave tokens out at both ends: those get zero gradients
        cu = [10, 90, 180]
        q, k, v, g, beta, do = (x[:1] for x in (q, k, v, g, beta, do))
        sl = slice(cu[0], cu[-1])
        ref = O.kda_grads(q[:, sl], k[:, sl], v[:, sl], g[:, sl], beta[:, sl], do[:, sl], dht, initial_state=h0,
                          cu_seqlens=[c - cu[0] for c in cu], dtype=torch.float32)
        _, _, got = _kda_grads_gpu(q, k, v, g, beta, h0, None, None, do, dht, cu=cu)
        for n in ('dq', 'dk', 'dv', 'dg', 'dbeta'):
            x = got[n]
            assert not x[:, :cu[0]].any() and not x[:, cu[-1]:].any(), f'{n}: tokens outside every sequence must get zero'
            got[n] = x[:, sl]
        _compare_grads(ref, got)
        return
    ref = O.kda_grads(q, k, v, g, beta, do, dht, initial_state=h0, dtype=torch.float32, **kw)
    _, _, got = _kda_grads_gpu(q, k, v, g, beta, h0, None, None, do, dht, **kw)
    _compare_grads(ref, got)


@pytest.mark.gpu
@pytest.mark.parametrize('packed,vfirst,V', [(False, False, 64), (True, False, 64), (False, True, 64), (False, False, 200)])
def test_chunk_kda_return_intermediate_states(packed, vfirst, V):
    """``return_intermediate_states`` (inference mode): the state in front of every chunk, against the oracle's final state of
    the tokens before that chunk (shapes and dtype as tests/ops/test_kda.py:1139-1211 of the reference)."""
    from fla_hip.ops.kda import chunk_kda
    B, T, H, HV, D = (1, 330, 2, 4, 64) if packed else (2, 200, 2, 4, 64)
    q, k, v, g, beta, h0, _, _ = _chunk_inputs(B, T, H, HV, D, 1.0, 0, False, False, torch.bfloat16, seed=11, V=V)
    cu = [0, 70, 70, 200, 330] if packed else None
    N = len(cu) - 1 if packed else B
    h0 = torch.randn(N, HV, D, V, generator=torch.Generator().manual_seed(12))
    d = lambda x: x.cuda()
    with torch.inference_mode():
        o, ht, h = chunk_kda(d(q), d(k), d(v), d(g), d(beta), initial_state=d(h0.transpose(-1, -2).contiguous() if vfirst else h0),
                             output_final_state=True, use_qk_l2norm_in_kernel=True, return_intermediate_states=True,
                             state_v_first=vfirst, cu_seqlens=None if cu is None else torch.tensor(cu, device='cuda'))
    bounds = [(0, s, e) for s, e in zip(cu[:-1], cu[1:])] if packed else [(b, 0, T) for b in range(B)]
    chunks = sum((e - s + 63) // 64 for _, s, e in bounds)
    nb = 1 if packed else B
    assert h.dtype == torch.bfloat16 and h.shape == (nb, chunks // nb, HV, *((V, D) if vfirst else (D, V)))
    hf = h.float().cpu().reshape(chunks, *h.shape[2:])
    c = 0
    for n, (b, s, e) in enumerate(bounds):
        for t0 in range(s, e, 64):
            sl = slice(s, t0)
            _, ref = O.recurrent_kda(q[b:b + 1, sl], k[b:b + 1, sl], v[b:b + 1, sl], g[b:b + 1, sl], beta[b:b + 1, sl], None, h0[n:n + 1], True,
                                     use_qk_l2norm_in_kernel=True)
            got = hf[c].transpose(-1, -2) if vfirst else hf[c]
            assert O.get_err_ratio(ref[0], got) < 0.005, (n, t0)
            c += 1
    assert c == chunks

