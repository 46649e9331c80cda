"""CPU-only tests: the C ABI library loads and exports what include/gdn_hip.h declares, and
the host logic (index tables, caches, guards, dispatch registry, argument validation, naive
torch forms) behaves like the reference's (tests/ops/utils/test_index.py, tests/ops/test_backends.py)."""
import ctypes
import os
import re

import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from fla_hip import _lib
    header = open(os.path.join(ROOT, 'include', 'gdn_hip.h')).read()
    header = re.sub(r'/\*.*?\*/', '', header, flags=re.S)
    declared = set(re.findall(r'\b(gdn_[a-z0-9_]+)\s*\(', header))
    assert declared == set(_lib.SIGNATURES), (declared, set(_lib.SIGNATURES))
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip('libgdn_hip.so not built in this checkout')
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f'{name} is declared in gdn_hip.h but missing from the library'
    assert _lib.load().gdn_hip_abi_version() == _lib.ABI_VERSION
    # pure host-side entry points can be called without a GPU
    l = _lib.load()
    ws = lambda N, T, NC, H, HV, K, V, packed=0, flags=0: l.gdn_chunk_workspace_bytes(N, T, NC, H, HV, K, V, packed, flags)
    assert ws(1, 512, 8, 2, 4, 128, 128) > 0
    assert ws(1, 512, 8, 2, 4, 64, 96) > 0          # multiples of 8 up to 128 are taken as they are
    assert ws(1, 512, 8, 2, 4, 100, 128) == 0
    # the segment matrices are reserved only when the plan cuts time into segments: long dense input with few heads
    rec = 12288 + 4                                 # a record and a transition bound per (chunk, value head)
    assert ws(1, 32768, 512, 16, 32, 128, 128) == 512 * 32 * rec + 3 * 8 * 32 * 65536
    assert ws(1, 32768, 512, 16, 32, 128, 128, 0, _lib.FLAG_SCAN_WIDE) == 512 * 32 * rec
    assert ws(32, 65536, 1040, 16, 32, 128, 128, 1) == 1040 * 32 * rec                 # packed input never does
    assert ws(64, 4096, 64 * 64, 16, 32, 128, 128) == 64 * 64 * 32 * rec               # enough runs already
    # argument errors are reported before any launch
    rc = l.gdn_fused_recurrent_fwd(1, 1, 1, None, None, None, None, None, None, None, None, 1, None, None, None, 1,
                                   1, 1, 2, 3, 64, 64, 1, 1.0, 0, 2, 0, None)
    assert rc == _lib.GDN_ERR_INVALID and 'divisible' in _lib.last_error()
    with pytest.raises(ValueError):
        _lib.check(rc)
    rc = l.gdn_fused_recurrent_fwd(1, 1, 1, None, None, None, None, None, None, None, None, 1, None, None, None, 1,
                                   1, 1, 1, 1, 512, 64, 1, 1.0, 0, 2, 0, None)
    assert rc == _lib.GDN_ERR_UNSUPPORTED
    with pytest.raises(NotImplementedError):
        _lib.check(rc)


def test_flag_and_status_constants_match_the_header():
    """The Python binding repeats the header's constants by value: they must agree, and no two flags
    may share a bit."""
    from fla_hip import _lib
    header = open(os.path.join(ROOT, 'include', 'gdn_hip.h')).read()
    flags = {n: (1 << int(b)) for n, b in re.findall(r'#define\s+GDN_FLAG_(\w+)\s+\(1u\s*<<\s*(\d+)\)', header)}
    assert len(flags) >= 11 and len(set(flags.values())) == len(flags)
    for name, value in flags.items():
        assert getattr(_lib, 'FLAG_' + name) == value, name
    m = re.search(r'#define\s+GDN_CHUNK_STATIC_WORKSPACE_BYTES\s+\((\d+)u\s*<<\s*(\d+)\)', header)
    assert int(m.group(1)) << int(m.group(2)) == _lib.CHUNK_STATIC_WORKSPACE_BYTES
    m = re.search(r'#define\s+GDN_CONV_BWD_TILES_PER_PART\s+(\d+)', header)
    assert int(m.group(1)) == _lib.CONV_BWD_TILES_PER_PART
    for name, value in re.findall(r'#define\s+(GDN_ERR_\w+|GDN_OK)\s+\(?(-?\d+)\)?', header):
        assert getattr(_lib, name) == int(value), name


@pytest.mark.parametrize('cu', [[0, 15], [0, 64], [0, 1, 65, 192, 193, 400], [0, 256, 500, 1000], [0, 100, 100, 164]])
@pytest.mark.parametrize('dtype', [torch.int64, torch.int32])
def test_chunk_tables_match_loop_reference(cu, dtype):
    from fla_hip.ops.utils.index import prepare_chunk_indices, prepare_chunk_offsets
    t = torch.tensor(cu, dtype=dtype)
    for cs in (16, 64):
        idx = prepare_chunk_indices(t, cs)
        assert idx.dtype == dtype and idx.tolist() == O.prepare_chunk_indices(cu, cs)
        off = prepare_chunk_offsets(t, cs)
        assert off.dtype == dtype and off.tolist() == O.prepare_chunk_offsets(cu, cs)
        # host copy gives the same table
        assert prepare_chunk_indices(t, cs, cu_seqlens_cpu=t.clone()).tolist() == idx.tolist()


def test_tensor_cache_is_by_identity():
    from fla_hip.utils import tensor_cache
    calls = []

    @tensor_cache
    def f(x, n):
        calls.append(1)
        return x * n

    a = torch.ones(3)
    r1 = f(a, 2)
    assert f(a, 2) is r1 and len(calls) == 1
    f(a.clone(), 2)                      # equal values, different object: recomputed
    assert len(calls) == 2
    f(a, n=2)                            # different call shape: recomputed
    assert len(calls) == 3
    # a tensor written in place since (a persistent buffer refilled by a serving loop) is not the tensor that was cached
    b = torch.ones(3)
    f(b, 2)
    f(b, 2)
    assert len(calls) == 4
    b.add_(1)
    assert f(b, 2).tolist() == [4.0, 4.0, 4.0] and len(calls) == 5
    # tensors made in inference mode have no version counter: calls with one are computed every time
    with torch.inference_mode():
        c = torch.ones(3)
        f(c, 2)
        c.add_(1)
        assert f(c, 2).tolist() == [4.0, 4.0, 4.0] and len(calls) == 7


def test_cu_seqlens_check_follows_in_place_updates():
    from fla_hip.ops.utils.index import check_cu_seqlens, prepare_chunk_indices
    cu = torch.tensor([0, 100, 200])
    check_cu_seqlens(cu, 200)
    assert prepare_chunk_indices(cu, 64).shape[0] == 4
    cu.copy_(torch.tensor([0, 100, 300]))            # same tensor object, new boundaries: checked and tabulated again
    with pytest.raises(ValueError):
        check_cu_seqlens(cu, 200)
    assert prepare_chunk_indices(cu, 64).shape[0] == 6


def test_input_guard_makes_contiguous():
    from fla_hip.utils import input_guard
    seen = {}

    @input_guard
    def f(x, y=None):
        seen['x'], seen['y'] = x.is_contiguous(), y.is_contiguous()
        return x

    @input_guard(no_guard_contiguous=['y'])
    def g(x, y=None):
        seen['x'], seen['y'] = x.is_contiguous(), y.is_contiguous()

    a = torch.randn(4, 6).t()
    f(a, y=a)
    assert seen == {'x': True, 'y': True}
    g(a, y=a)
    assert seen == {'x': True, 'y': False}


def test_dispatch_registry_priority_verifier_and_fallthrough(monkeypatch):
    from fla_hip.ops.backends import BackendRegistry, BaseBackend, dispatch
    reg = BackendRegistry('unit_test_op')
    BackendRegistry._initialized.add('unit_test_op')
    log = []

    @dispatch('unit_test_op')
    def op(x, flag=False):
        log.append('default')
        return x

    class Low(BaseBackend):
        backend_type, priority = 'low', 7

        def op(self, x, flag=False):
            log.append('low')
            return x + 1

    class High(BaseBackend):
        backend_type, priority = 'high', 2

        def op_verifier(self, x, flag=False):
            if flag:
                raise RuntimeError('boom')       # a raising verifier is a rejection
            return x < 10, 'x too large'

        def op(self, x, flag=False):
            log.append('high')
            return x + 100

    class Gated(BaseBackend):
        backend_type, priority, env_var, default_enable = 'gated', 0, 'UNIT_TEST_GATED', False

        def op(self, x, flag=False):
            log.append('gated')
            return -1

    class Missing(BaseBackend):
        backend_type, priority, package_name = 'missing', 0, 'surely_not_an_installed_package_xyz'

        def op(self, x, flag=False):
            return -2

    for b in (Low(), High(), Gated(), Missing()):
        reg.register(b)
    assert op(1) == 101 and log[-1] == 'high'             # lowest priority number wins
    assert op(50) == 51 and log[-1] == 'low'              # verifier rejects -> next backend
    assert op(1, flag=True) == 2 and log[-1] == 'low'     # verifier raised -> rejected, not an error
    monkeypatch.setenv('UNIT_TEST_GATED', '1')
    assert op(1) == -1 and log[-1] == 'gated'             # env var opts the gated backend in
    monkeypatch.delenv('UNIT_TEST_GATED')
    assert reg.get_active().backend_type == 'high'
    # an operation without backends falls through to the decorated default
    @dispatch('unit_test_op_without_backends')
    def op2(x):
        return x * 2
    assert op2(4) == 8
    from fla_hip.ops.gated_delta_rule.backends import gated_delta_rule_registry
    assert gated_delta_rule_registry.operation_name == 'gated_delta_rule'


def test_public_surface_and_signatures():
    import inspect
    import importlib
    pkg = importlib.import_module('flash-linear-attention_amd')
    import fla_hip.ops.gated_delta_rule as m
    assert m.__all__ == ['chunk_gated_delta_rule', 'chunk_gdn', 'fused_recurrent_gated_delta_rule', 'fused_recurrent_gdn',
                         'naive_chunk_gated_delta_rule', 'naive_recurrent_gated_delta_rule']
    assert pkg.chunk_gdn is m.chunk_gated_delta_rule and m.fused_recurrent_gdn is m.fused_recurrent_gated_delta_rule
    # parameter names are ABI (callers filter keyword arguments by name)
    assert list(inspect.signature(m.chunk_gated_delta_rule).parameters) == [
        'q', 'k', 'v', 'g', 'beta', 'scale', 'initial_state', 'output_final_state', 'use_qk_l2norm_in_kernel',
        'use_beta_sigmoid_in_kernel', 'allow_neg_eigval', 'state_v_first', 'cu_seqlens', 'cu_seqlens_cpu',
        'chunk_indices', 'cp_context', 'kwargs']
    assert list(inspect.signature(m.fused_recurrent_gated_delta_rule).parameters) == [
        'q', 'k', 'v', 'g', 'gk', 'gv', 'beta', 'scale', 'initial_state', 'output_final_state',
        'use_qk_l2norm_in_kernel', 'use_gate_in_kernel', 'A_log', 'dt_bias', 'use_beta_sigmoid_in_kernel',
        'allow_neg_eigval', 'state_v_first', 'cu_seqlens', 'kwargs']
    assert list(inspect.signature(m.naive_recurrent_gated_delta_rule).parameters)[:5] == ['q', 'k', 'v', 'beta', 'g']
    assert list(inspect.signature(m.naive_chunk_gated_delta_rule).parameters)[:5] == ['q', 'k', 'v', 'g', 'beta']


def test_validation_happens_on_the_host_and_cpu_tensors_are_refused():
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule
    q = torch.randn(2, 8, 2, 16)
    v = torch.randn(2, 8, 4, 16)
    g = torch.zeros(2, 8, 4)
    with pytest.raises(ValueError, match='same number of heads'):
        chunk_gated_delta_rule(q, q[:, :, :1], v, g, g)
    with pytest.raises(ValueError, match='divisible'):
        chunk_gated_delta_rule(q, q, v[:, :, :3], g[:, :, :3], g[:, :, :3])
    with pytest.raises(ValueError, match='chunk_size'):
        chunk_gated_delta_rule(q, q, v, g, g, chunk_size=128)
    with pytest.raises(ValueError, match='batch size'):
        chunk_gated_delta_rule(q, q, v, g, g, cu_seqlens=torch.tensor([0, 8, 16]))
    with pytest.raises(ValueError, match='initial states'):
        chunk_gated_delta_rule(q[:1], q[:1], v[:1], g[:1], g[:1], initial_state=torch.zeros(3, 4, 16, 16),
                               cu_seqlens=torch.tensor([0, 4, 8]))
    with pytest.raises(ValueError, match='allow_neg_eigval'):
        chunk_gated_delta_rule(q, q, v, g, g, allow_neg_eigval=True)
    with pytest.raises(AssertionError, match='A_log'):
        chunk_gated_delta_rule(q, q, v, g, g, use_gate_in_kernel=True)
    with pytest.raises(DeprecationWarning):
        chunk_gated_delta_rule(q, q, v, g, g, head_first=False)
    with pytest.raises(ValueError, match='transpose_state_layout'):
        chunk_gated_delta_rule(q, q, v, g, g, state_v_first=True, transpose_state_layout=True)
    with pytest.raises(NotImplementedError):
        chunk_gated_delta_rule(q, q, v, g, g, cp_context=object())
    with pytest.raises(ValueError, match='A_log'):
        fused_recurrent_gated_delta_rule(q, q, v, g, use_gate_in_kernel=True)
    with pytest.raises(ValueError, match='inplace_final_state'):
        fused_recurrent_gated_delta_rule(q, q, v, g, inplace_final_state=True)
    # no CPU or eager fallback exists: CPU tensors are an error, not a slow path
    with pytest.raises(RuntimeError, match='ROCm GPU'):
        chunk_gated_delta_rule(q, q, v, g, g)
    with pytest.raises(RuntimeError, match='ROCm GPU'):
        fused_recurrent_gated_delta_rule(q, q, v, g)


def test_naive_forms_match_oracle():
    from fla_hip.ops.gated_delta_rule import naive_chunk_gated_delta_rule, naive_recurrent_gated_delta_rule
    q, k, v, g, beta, h0 = O.make_inputs(2, 150, 2, 2, 16, 8, seed=13, h0_std=0.5)
    ref_o, ref_h = O.recurrent_gated_delta_rule(q, k, v, g, beta, None, h0, True, dtype=torch.float64)
    o1, h1 = naive_recurrent_gated_delta_rule(q, k, v, beta, g, initial_state=h0, output_final_state=True)
    o2, h2 = naive_chunk_gated_delta_rule(q, k, v, g, beta, initial_state=h0, output_final_state=True)
    for o, h in ((o1, h1), (o2, h2)):
        assert o.shape == ref_o.shape
        assert O.get_err_ratio(ref_o, o) < 1e-5 and O.get_err_ratio(ref_h, h) < 1e-5
    o3, h3 = naive_chunk_gated_delta_rule(q, k, v, g, beta, chunk_size=16, scale=0.3)
    ref_o3, _ = O.recurrent_gated_delta_rule(q, k, v, g, beta, 0.3, dtype=torch.float64)
    assert h3 is None and O.get_err_ratio(ref_o3, o3) < 1e-5


def test_naive_comba_forms():
    """The chunked plain-torch form is the oracle's recurrence (predict before the decay); the token loop of that name decays
    first, as the reference's does, and equals the chunked form only where there is no decay."""
    from fla_hip.ops.comba import naive_chunk_comba, naive_recurrent_comba
    gen = torch.Generator().manual_seed(17)
    q, k, p = (F.normalize(torch.randn(2, 150, 2, 16, generator=gen), dim=-1) for _ in range(3))
    v = torch.randn(2, 150, 2, 8, generator=gen)
    g = F.logsigmoid(torch.randn(2, 150, 2, generator=gen))
    beta = torch.rand(2, 150, 2, generator=gen)
    h0 = torch.randn(2, 2, 16, 8, generator=gen)
    ref_o, ref_h = O.recurrent_comba(q, k, v, p, g, beta, None, h0, True, dtype=torch.float64)
    for cs in (64, 16):
        o, h = naive_chunk_comba(q, k, v, p, g, beta, chunk_size=cs, initial_state=h0, output_final_state=True)
        assert o.shape == ref_o.shape and O.get_err_ratio(ref_o, o) < 1e-5 and O.get_err_ratio(ref_h, h) < 1e-5
    o_r, h_r = naive_recurrent_comba(q, k, v, p, beta, g, initial_state=h0, output_final_state=True)
    assert O.get_err_ratio(ref_o, o_r) > 1e-3                                         # (a different map)
    zero = torch.zeros_like(g)
    o_r0, h_r0 = naive_recurrent_comba(q, k, v, p, beta, zero, initial_state=h0, output_final_state=True)
    ref0, refh0 = O.recurrent_comba(q, k, v, p, zero, beta, None, h0, True, dtype=torch.float64)
    assert O.get_err_ratio(ref0, o_r0) < 1e-5 and O.get_err_ratio(refh0, h_r0) < 1e-5
    # its decay-first step in scalars: S <- e^g S, then the delta rule with p
    S = h0[0, 0].double() * g[0, 0, 0].exp().double()
    d = beta[0, 0, 0].double() * (v[0, 0, 0].double() - S.T @ p[0, 0, 0].double())
    S = S + torch.outer(k[0, 0, 0].double(), d)
    assert torch.allclose(o_r[0, 0, 0].double(), (S.T @ q[0, 0, 0].double()) * 16 ** -0.5, atol=1e-5)


def test_assert_close_metric():
    from fla_hip.utils import assert_close, get_abs_err, get_err_ratio
    x = torch.tensor([3.0, 4.0]); y = torch.tensor([3.0, 5.0])
    assert get_abs_err(x, y) == 1.0 and abs(get_err_ratio(x, y) - O.get_err_ratio(x, y)) < 1e-6
    assert_close('ok', x, x + 1e-7, 1e-6)
    with pytest.raises(AssertionError):
        assert_close('bad', x, y, 0.01)
    with pytest.warns(UserWarning):
        assert_close('warn', x, y, 0.01, warning=True)


def test_scan_tables_offsets_then_longest_first_order():
    """prepare_scan_tables = prepare_chunk_offsets followed by the sequence ids by decreasing
    number of chunks (ties keep packed order)."""
    import torch
    from fla_hip.ops.utils.index import prepare_chunk_offsets, prepare_scan_tables
    cu = torch.tensor([0, 5, 300, 301, 1000, 1064, 1064 + 700])
    t = prepare_scan_tables(cu, 64)
    n = cu.numel() - 1
    assert t.dtype == cu.dtype and t.numel() == 2 * n + 1
    assert torch.equal(t[:n + 1], prepare_chunk_offsets(cu, 64))
    counts = [(int(b - a) + 63) // 64 for a, b in zip(cu[:-1], cu[1:])]
    order = t[n + 1:].tolist()
    assert sorted(order) == list(range(n))
    assert [counts[i] for i in order] == sorted(counts, reverse=True)
    assert order == sorted(range(n), key=lambda i: (-counts[i], i))


def test_upstream_backends_follow_the_plugin_interface():
    # the backends for an unmodified upstream fla, exercised through this package's mirror of the registry:
    # CPU tensors are rejected by the verifier, so the decorated default runs
    import torch
    from fla_hip.ops.backends import BackendRegistry, BaseBackend, dispatch
    from fla_hip.upstream import make_backends
    op_cls, mod_cls = make_backends(BaseBackend)
    assert issubclass(op_cls, BaseBackend) and op_cls.priority < 3 and op_cls.package_name == 'fla_hip'
    assert op_cls.is_available() and op_cls.is_enabled()
    reg = BackendRegistry('upstream_test_cpu')
    reg.register(op_cls())
    calls = []

    @dispatch('upstream_test_cpu')
    def chunk_gated_delta_rule(q, k, v, g, beta, **kwargs):
        calls.append('default')
        return 'default'

    x = torch.zeros(1, 4, 1, 8)
    assert chunk_gated_delta_rule(x, x, x, x[..., 0], x[..., 0]) == 'default' and calls == ['default']
    be = mod_cls()
    for name in ('causal_conv1d_fwd', 'causal_conv1d_bwd', 'causal_conv1d_update_states', 'causal_conv1d_update', 'layer_norm_gated_fwd',
                 'layer_norm_gated_bwd'):
        assert callable(getattr(be, name)) and callable(getattr(be, name + '_verifier'))
    assert be.verify('causal_conv1d_fwd', x[0], torch.zeros(8, 4))[0] is False
    assert be.verify('layer_norm_gated_fwd', x[0, :, 0], x[0, :, 0], None, None)[0] is False
    assert be.verify('causal_conv1d_bwd', x[0], x[0], None, torch.zeros(8, 4))[0] is False
    assert be.verify('layer_norm_gated_bwd', x[0, :, 0], x[0, :, 0], x[0, :, 0], None, None)[0] is False
    os.environ['FLA_HIP_GFX950'] = '0'
    try:
        assert not op_cls.is_enabled()
    finally:
        del os.environ['FLA_HIP_GFX950']


@pytest.mark.gpu
def test_upstream_backends_take_gpu_inference_calls_and_leave_the_rest():
    import torch
    from fla_hip.ops.backends import BackendRegistry, BaseBackend, dispatch
    from fla_hip.upstream import make_backends
    from oracle import gdn_oracle as O
    op_cls, mod_cls = make_backends(BaseBackend)
    BackendRegistry('upstream_test_gpu').register(op_cls())
    BackendRegistry('upstream_test_modules').register(mod_cls())

    @dispatch('upstream_test_gpu')
    def chunk_gated_delta_rule(q, k, v, g, beta, **kwargs):
        return 'default', None

    @dispatch('upstream_test_modules')
    def causal_conv1d_fwd(x, weight, bias, residual, initial_state=None, output_final_state=False, activation=None, **kwargs):
        return 'default', None

    @dispatch('upstream_test_modules')
    def layer_norm_gated_fwd(x, g, weight, bias, activation='swish', eps=1e-5, residual=None, out_dtype=None,
                             residual_dtype=None, is_rms_norm=False):
        return 'default'

    q, k, v, g, beta, _ = O.make_inputs(1, 130, 2, 4, 64, 64, seed=3, dtype=torch.bfloat16)
    ref, _ = O.chunk_gated_delta_rule(q, k, v, g, beta, None, None, False)
    dq, dk, dv, dg, db = (t.cuda() for t in (q, k, v, g, beta))
    o, ht = chunk_gated_delta_rule(dq, dk, dv, dg, db, output_final_state=False)
    assert isinstance(o, torch.Tensor) and ht is None and O.get_err_ratio(ref, o.float().cpu()) < 5e-3
    o_t = chunk_gated_delta_rule(dq.requires_grad_(), dk, dv, dg, db)[0]                          # training goes through the backward kernels
    assert isinstance(o_t, torch.Tensor) and o_t.requires_grad
    assert chunk_gated_delta_rule(q, k, v, g, beta)[0] == 'default'                               # CPU stays upstream
    # fp32 operands stay upstream too (it multiplies them as tf32; the chunk kernels here would round them to bf16)
    assert chunk_gated_delta_rule(dq.detach().float(), dk.float(), dv.float(), dg, db)[0] == 'default'
    with torch.no_grad():
        assert isinstance(chunk_gated_delta_rule(dq, dk, dv, dg, db)[0], torch.Tensor)
    x = torch.randn(2, 40, 64, device='cuda', dtype=torch.bfloat16)
    w = torch.randn(64, 4, device='cuda', dtype=torch.bfloat16)
    y, st = causal_conv1d_fwd(x, w, None, None, activation='silu', output_final_state=True)
    assert y.shape == x.shape and st.shape == (2, 64, 4)
    assert causal_conv1d_fwd(x, torch.randn(64, 9, device='cuda', dtype=torch.bfloat16), None, None)[0] == 'default'
    assert causal_conv1d_fwd(x, w, None, None, activation='gelu')[0] == 'default'
    out = layer_norm_gated_fwd(x[0], x[1], None, None, is_rms_norm=True)
    assert len(out) == 4 and out[0].shape == x[0].shape and out[1] is None
    assert layer_norm_gated_fwd(x[0], x[1], None, None, activation='relu') == 'default'

    # the backward entries upstream's autograd functions call (fla/modules/conv/triton/ops.py:411-428, fla/modules/fused_norm_gate.py:712-733)
    @dispatch('upstream_test_modules')
    def causal_conv1d_bwd(x, dy, dht, weight=None, bias=None, residual=None, initial_state=None, activation=None, **kwargs):
        return ('default',) * 5

    @dispatch('upstream_test_modules')
    def layer_norm_gated_bwd(dy, x, g, weight, bias, activation='swish', eps=1e-5, mean=None, rstd=None, dresidual=None,
                             has_residual=False, is_rms_norm=False, x_dtype=None, recompute_output=False):
        return ('default',) * 5

    dx, dw, db_, dr, dh0 = causal_conv1d_bwd(x, torch.randn_like(x), None, weight=w, activation='silu')
    assert dx.shape == x.shape and dw.shape == w.shape and db_ is None and dr is None and dh0 is None
    assert causal_conv1d_bwd(x, torch.randn_like(x), None, weight=w, activation='gelu')[0] == 'default'
    grads = layer_norm_gated_bwd(x[0], x[0], x[1], None, None, rstd=out[2], is_rms_norm=True)
    assert grads[0].shape == x[0].shape and grads[2] is None and grads[4] is None
    assert layer_norm_gated_bwd(x[0], x[0], x[1], None, None, rstd=out[2], is_rms_norm=True, recompute_output=True)[0] == 'default'


def test_operand_shapes_are_checked_before_anything_reaches_a_kernel():
    """g, beta, gk, gv of a shape other than the one q and v imply would be read out of bounds by the kernels: the host
    refuses them (the helper itself needs no GPU)."""
    import torch
    from fla_hip.ops.gated_delta_rule._common import check_operand_shapes
    q = torch.zeros(2, 8, 2, 16)
    v = torch.zeros(2, 8, 4, 32)
    g = torch.zeros(2, 8, 4)
    check_operand_shapes(q, q, v, g=g, beta=g, gk=torch.zeros(2, 8, 4, 16), gv=torch.zeros(2, 8, 4, 32))
    check_operand_shapes(q, q, v, g=g[..., None], beta=torch.zeros(2, 8, 4, 32), beta_per_column=True)
    for bad in (dict(g=torch.zeros(2, 8, 2)), dict(beta=torch.zeros(2, 8, 4, 32)), dict(gk=g), dict(gk=torch.zeros(2, 8, 4, 32)),
                dict(gv=torch.zeros(2, 8, 4, 16)), dict(beta=torch.zeros(2, 7, 4))):
        with pytest.raises(ValueError, match='must have shape'):
            check_operand_shapes(q, q, v, **bad)
    with pytest.raises(ValueError, match='same shape'):
        check_operand_shapes(q, q[..., :8], v)
    with pytest.raises(ValueError, match='batch and sequence'):
        check_operand_shapes(q, q, v[:, :4])
    with pytest.raises(ValueError, match='divisible'):
        check_operand_shapes(q, q, v[:, :, :3])


def test_cu_seqlens_are_checked_on_the_host_copy():
    import torch
    from fla_hip.ops.utils.index import check_cu_seqlens
    check_cu_seqlens(torch.tensor([0, 3, 3, 10]), 10)
    check_cu_seqlens(torch.tensor([2, 5], dtype=torch.int32), 10)                   # tokens outside all sequences are allowed
    check_cu_seqlens(torch.tensor([0, 99]), 10, cu_seqlens_cpu=torch.tensor([0, 10]))      # (the host copy is what is read)
    for bad in ([0, 11], [-1, 4], [0, 6, 5, 10], [0]):
        with pytest.raises(ValueError, match='cu_seqlens must'):
            check_cu_seqlens(torch.tensor(bad), 10)


@pytest.mark.gpu
def test_packed_calls_refuse_boundaries_beyond_the_input():
    import torch
    from fla_hip.modules import causal_conv1d
    from fla_hip.ops.comba import chunk_comba
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    from fla_hip.ops.kda import chunk_kda
    q = torch.randn(1, 100, 2, 64, device='cuda', dtype=torch.bfloat16)
    g = -torch.rand(1, 100, 2, device='cuda')
    cu = torch.tensor([0, 50, 101], device='cuda')
    with pytest.raises(ValueError, match='cu_seqlens must'):
        chunk_gated_delta_rule(q, q, q, g, g.exp(), cu_seqlens=cu)
    with pytest.raises(ValueError, match='cu_seqlens must'):
        chunk_gated_delta_rule(q.clone().requires_grad_(), q, q, g, g.exp(), cu_seqlens=torch.tensor([0, 60, 40, 100], device='cuda'))
    with pytest.raises(ValueError, match='cu_seqlens must'):
        chunk_kda(q, q, q, g[..., None].expand(-1, -1, -1, 64).contiguous(), g.exp(), cu_seqlens=cu)
    with pytest.raises(ValueError, match='cu_seqlens must'):
        chunk_comba(q, q, q, q, g, g.exp(), cu_seqlens=cu)
    x = torch.randn(1, 100, 64, device='cuda', dtype=torch.bfloat16, requires_grad=True)
    y, _ = causal_conv1d(x, torch.randn(64, 4, device='cuda', dtype=torch.bfloat16), cu_seqlens=torch.tensor([0, 100], device='cuda'))
    y.sum().backward()
    assert x.grad is not None
