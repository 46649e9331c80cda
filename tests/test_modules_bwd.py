"""Backward of the convolution and the gated normalisation on the GPU (gdn_causal_conv1d_bwd, gdn_norm_gated_bwd through
fla_hip.modules' autograd functions) against the CPU oracle's gradients, on the matrices of the reference's own tests
(tests/modules/test_conv.py:118-275 dense and packed, :960-1100 initial-state gradients; tests/modules/test_layernorm_gated.py:
20-110).

Tolerances as for the forward: the oracle is the exact formula on the rounded inputs, what remains is the rounding of each
gradient to its dtype and fp32 summation order: rel-RMSE <= 3e-3 (bf16), 5e-4 (fp16), 5e-6 (fp32); the reference's tests use 1e-3."""
import pytest
import torch

from oracle import modules_oracle as M
from oracle.gdn_oracle import get_err_ratio

pytestmark = pytest.mark.gpu

DEV = 'cuda'
TOL = {torch.float32: 5e-6, torch.float16: 5e-4, torch.bfloat16: 3e-3}


def _mods():
    import fla_hip.modules as mods
    return mods


def _close(name, ref, tri, dtype):
    assert tri is not None, name
    assert tri.dtype == dtype, (name, tri.dtype)
    assert tuple(tri.shape) == tuple(ref.shape), (name, tri.shape, ref.shape)
    err = get_err_ratio(ref.double(), tri.double().cpu())
    assert err <= TOL[dtype], f'{name}: rel-RMSE {err:.3e} > {TOL[dtype]:.1e}'


def _conv_case(B, T, D, W, dtype, has_bias, has_residual, state=False, N=None, seed=42):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(B, T, D, generator=gen).to(dtype)
    w = torch.randn(D, W, generator=gen).to(dtype)
    b = torch.randn(D, generator=gen).to(dtype) if has_bias else None
    r = torch.randn(B, T, D, generator=gen).to(dtype) if has_residual else None
    s = torch.randn(N or B, D, W, generator=gen).to(dtype) if state else None
    dy = torch.randn(B, T, D, generator=gen).to(dtype)
    dht = torch.randn(N or B, D, W, generator=gen).to(dtype) if state else None
    return x, w, b, r, s, dy, dht


def _run_conv(x, w, b, r, s, dy, dht, activation, cu=None, cu_dtype=torch.int64):
    leaves = [None if t is None else t.to(DEV).requires_grad_(True) for t in (x, w, b, r, s)]
    cu_t = None if cu is None else torch.tensor(cu, dtype=cu_dtype, device=DEV)
    y, final = _mods().causal_conv1d(leaves[0], leaves[1], leaves[2], leaves[3], leaves[4], dht is not None, activation, cu_seqlens=cu_t)
    loss = (y.float() * dy.to(DEV).float()).sum()
    if dht is not None:
        loss = loss + (final.float() * dht.to(DEV).float()).sum()
    loss.backward()
    return y, [None if t is None else t.grad for t in leaves]


def _check_conv(case, activation, cu=None, cu_dtype=torch.int64):
    x, w, b, r, s, dy, dht = case
    ref = M.conv_grads(x, w, b, r, s, dy, dht, activation, cu)
    ref_y, _ = M.causal_conv1d(x, w, b, r, s, False, activation, cu)
    y, (dx, dw, db, dr, dh0) = _run_conv(x, w, b, r, s, dy, dht, activation, cu, cu_dtype)
    dtype = x.dtype
    _close('y', ref_y, y.detach(), dtype)
    _close('dx', ref['dx'], dx, dtype)
    _close('dw', ref['dw'], dw, dtype)
    if b is not None:
        _close('db', ref['db'], db, dtype)
    if r is not None:
        _close('dr', ref['dr'], dr, dtype)
    if s is not None:
        _close('dh0', ref['dh0'], dh0, dtype)


DENSE = [
    (2, 64, 128, 3, 'swish', True, True, torch.float32),
    (2, 128, 128, 4, 'swish', False, True, torch.float32),
    (2, 64, 128, 3, 'swish', True, False, torch.float32),
    (2, 128, 128, 4, 'swish', False, False, torch.float32),
    (2, 500, 1024, 3, None, True, True, torch.float32),
    (2, 1024, 1024, 4, None, False, True, torch.float32),
    (2, 64, 128, 3, None, True, False, torch.float16),
    (2, 128, 128, 4, None, False, False, torch.float16),
    (2, 500, 1024, 4, 'silu', True, True, torch.bfloat16),
    (3, 77, 200, 2, 'silu', False, False, torch.bfloat16),
    (1, 33, 100, 7, None, True, False, torch.bfloat16),
    (2, 50, 77, 4, 'silu', True, True, torch.bfloat16),        # an odd number of channels: padded on the host
    (2, 40, 64, 1, 'silu', True, False, torch.float16),
    (2, 40, 64, 8, 'silu', False, True, torch.float32),
]


@pytest.mark.parametrize(('B', 'T', 'D', 'W', 'activation', 'has_bias', 'has_residual', 'dtype'), DENSE)
def test_conv_backward_dense(B, T, D, W, activation, has_bias, has_residual, dtype):
    _check_conv(_conv_case(B, T, D, W, dtype, has_bias, has_residual), activation)


def _cu(N, T, seed=0):
    gen = torch.Generator().manual_seed(seed)
    cuts = torch.randperm(T - 1, generator=gen)[:N - 1].add(1).sort().values.tolist()
    return [0] + cuts + [T]


@pytest.mark.parametrize(('N', 'T', 'D', 'W', 'activation', 'has_bias', 'has_residual', 'dtype', 'cu_dtype'), [
    (4, 500, 128, 3, 'swish', True, True, torch.float32, torch.int64),       # tests/modules/test_conv.py:197-210
    (4, 1024, 200, 4, 'swish', False, True, torch.float32, torch.int32),
    (4, 500, 128, 3, None, True, False, torch.float16, torch.int64),
    (3, 1024, 256, 4, None, False, False, torch.bfloat16, torch.int32),
    (9, 300, 64, 4, 'silu', True, False, torch.bfloat16, torch.int64),
])
def test_conv_backward_packed(N, T, D, W, activation, has_bias, has_residual, dtype, cu_dtype):
    _check_conv(_conv_case(1, T, D, W, dtype, has_bias, has_residual), activation, _cu(N, T), cu_dtype)


@pytest.mark.parametrize('activation', [None, 'silu'])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_conv_backward_with_states(activation, dtype):
    """Initial state and the gradient of the final state, dense and packed; sequences shorter than the kernel (their initial
    state reaches the final state), an empty one, and tokens outside all sequences (zero gradient)."""
    _check_conv(_conv_case(3, 130, 64, 4, dtype, True, True, state=True), activation)
    _check_conv(_conv_case(2, 2, 64, 4, dtype, False, False, state=True), activation)
    cu = [0, 1, 1, 3, 70, 200]
    _check_conv(_conv_case(1, 200, 64, 4, dtype, True, False, state=True, N=5), activation, cu)
    cu = [5, 64, 128, 190]
    case = _conv_case(1, 200, 64, 3, dtype, True, True, state=True, N=3)
    x, w, b, r, s, dy, dht = case
    _, (dx, dw, db, dr, dh0) = _run_conv(x, w, b, r, s, dy, dht, activation, cu)
    assert dx[:, :5].abs().max() == 0 and dx[:, 190:].abs().max() == 0
    # (the oracle's packed form covers [cu[0], cu[N]); the tokens outside carry no gradient into the taps either)
    ref = M.conv_grads(x, w, b, r, s, dy, dht, activation, cu)
    _close('dx', ref['dx'], dx, dtype)
    _close('dw', ref['dw'], dw, dtype)
    _close('dh0', ref['dh0'], dh0, dtype)


@pytest.mark.parametrize('W', [2, 4, 7])
@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float32])
def test_conv_backward_long_runs(W, dtype):
    """Several runs of eight tiles per workgroup, so that most waves take the loop for runs inside one sequence: dense rows
    whose boundaries fall inside a run, and packed sequences that start, end and hand over a final-state gradient inside runs
    (lengths that are and are not multiples of the tile and of the strip)."""
    _check_conv(_conv_case(2, 1600, 96, W, dtype, True, False, state=True), 'silu')
    cu = [0, 700, 701, 1340, 1344, 2368, 3000]
    _check_conv(_conv_case(1, 3000, 72, W, dtype, False, True, state=True, N=6), 'silu', cu, torch.int32)
    _check_conv(_conv_case(1, 3000, 72, W, dtype, True, False, state=False), None, cu, torch.int64)


def test_conv_backward_reads_a_slice_in_place_and_is_deterministic():
    gen = torch.Generator().manual_seed(3)
    wide = torch.randn(2, 300, 3 * 256, generator=gen).bfloat16()
    x = wide[..., 256:512]
    _, w, b, _, _, dy, _ = _conv_case(2, 300, 256, 4, torch.bfloat16, True, False)
    ref = M.conv_grads(x, w, b, None, None, dy, None, 'silu')
    wide_d = wide.to(DEV).requires_grad_(True)
    w_d, b_d = w.to(DEV).requires_grad_(True), b.to(DEV).requires_grad_(True)
    outs = []
    for _ in range(2):
        y, _ = _mods().causal_conv1d(wide_d[..., 256:512], w_d, b_d, activation='silu')
        outs.append(torch.autograd.grad((y.float() * dy.to(DEV).float()).sum(), (wide_d, w_d, b_d)))
    assert all(torch.equal(a, c) for a, c in zip(*outs))
    dwide, dw, db = outs[0]
    assert dwide[..., :256].abs().max() == 0 and dwide[..., 512:].abs().max() == 0
    _close('dx', ref['dx'], dwide[..., 256:512], torch.bfloat16)
    _close('dw', ref['dw'], dw, torch.bfloat16)
    _close('db', ref['db'], db, torch.bfloat16)


def test_short_convolution_layer_trains():
    mods = _mods()
    conv = mods.ShortConvolution(128, 4, bias=True, activation='silu', device=DEV, dtype=torch.bfloat16)
    gen = torch.Generator().manual_seed(4)
    x = torch.randn(2, 100, 128, generator=gen).bfloat16()
    dy = torch.randn(2, 100, 128, generator=gen).bfloat16()
    xd = x.to(DEV).requires_grad_(True)
    y, _ = conv(xd)
    y.backward(dy.to(DEV))
    ref = M.conv_grads(x, conv.weight.detach().squeeze(1).cpu(), conv.bias.detach().cpu(), None, None, dy, None, 'silu')
    _close('dx', ref['dx'], xd.grad, torch.bfloat16)
    _close('dw', ref['dw'], conv.weight.grad.squeeze(1), torch.bfloat16)
    _close('db', ref['db'], conv.bias.grad, torch.bfloat16)
    # the one-token step stays forward only
    with pytest.raises(NotImplementedError, match='no backward'):
        conv.step(xd[:, :1], None, torch.zeros(2, 128, 4, device=DEV, dtype=torch.bfloat16))


# --------------------------------------------------------------------------- #
# gated normalisation
# --------------------------------------------------------------------------- #
def _check_norm(T_shape, D, dtype, affine, bias, activation, is_rms, residual=False, prenorm=False, fp32_stream=False, seed=42):
    mods = _mods()
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(*T_shape, D, generator=gen).to(dtype)
    g = torch.randn(*T_shape, D, generator=gen).to(dtype)
    res = torch.randn(*T_shape, D, generator=gen).to(torch.float32 if fp32_stream else dtype) if residual else None
    dy = torch.randn(*T_shape, D, generator=gen).to(dtype)
    dres = torch.randn(*T_shape, D, generator=gen).to(torch.float32 if fp32_stream else dtype) if prenorm else None
    w = torch.randn(D, generator=gen).to(dtype) if affine else None
    b = torch.randn(D, generator=gen).to(dtype) if bias else None
    leaves = [None if t is None else t.to(DEV).requires_grad_(True) for t in (x, g, w, b, res)]
    fn = mods.rms_norm_gated if is_rms else mods.layer_norm_gated
    out = fn(leaves[0], leaves[1], leaves[2], leaves[3], activation, leaves[4], prenorm, fp32_stream, 1e-5)
    y, r_out = out if prenorm else (out, None)
    loss = (y.float() * dy.to(DEV).float()).sum()
    if prenorm:
        loss = loss + (r_out.float() * dres.to(DEV).float()).sum()
    loss.backward()
    flat = lambda t: None if t is None else t.reshape(-1, D)
    ref = M.norm_gated_grads(flat(x), flat(g), w, b, flat(res), flat(dy), flat(dres), 1e-5, activation, is_rms)
    ref_y, _, _, _ = M.norm_gated(flat(x), flat(g), w, b, flat(res), 1e-5, activation, is_rms)
    _close('y', ref_y.reshape(*T_shape, D), y.detach(), dtype)
    _close('dx', ref['dx'].reshape(*T_shape, D), leaves[0].grad, dtype)
    _close('dg', ref['dg'].reshape(*T_shape, D), leaves[1].grad, dtype)
    if affine:
        _close('dw', ref['dw'], leaves[2].grad, dtype)
    if bias:
        _close('db', ref['db'], leaves[3].grad, dtype)
    if residual:
        _close('dr', ref['dr'].reshape(*T_shape, D), leaves[4].grad, res.dtype)


@pytest.mark.parametrize(('B', 'H', 'T', 'D', 'affine', 'activation', 'bias'), [
    (2, 2, 1, 64, False, 'silu', False),                        # tests/modules/test_layernorm_gated.py:25-30
    (2, 2, 512, 128, True, 'silu', True),
    (2, 2, 2048, 1200, True, 'sigmoid', False),
    (2, 2, 50, 50, False, 'sigmoid', False),
])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_layer_norm_gated_backward(B, H, T, D, affine, activation, bias, dtype):
    _check_norm((B, H, T), D, dtype, affine, bias, activation, False)


@pytest.mark.parametrize(('B', 'H', 'T', 'D', 'activation'), [
    (2, 2, 1, 64, 'silu'),                                      # tests/modules/test_layernorm_gated.py:66-71
    (2, 2, 512, 128, 'sigmoid'),
    (2, 2, 2048, 1200, 'silu'),
    (2, 2, 50, 50, 'sigmoid'),
    (4, 1, 1000, 256, 'swish'),
])
@pytest.mark.parametrize('dtype', [torch.float32, torch.float16, torch.bfloat16])
def test_rms_norm_gated_backward(B, H, T, D, activation, dtype):
    _check_norm((B, H, T), D, dtype, True, False, activation, True)


@pytest.mark.parametrize('is_rms', [False, True])
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
def test_norm_gated_backward_residual_stream(is_rms, dtype):
    _check_norm((3, 70), 128, dtype, True, not is_rms, 'swish', is_rms, residual=True)
    _check_norm((3, 70), 128, dtype, True, False, 'swish', is_rms, residual=True, prenorm=True)
    _check_norm((3, 70), 96, dtype, True, False, 'sigmoid', is_rms, residual=True, prenorm=True, fp32_stream=True)


def test_norm_gated_layer_trains_and_limits():
    mods = _mods()
    norm = mods.FusedRMSNormGated(128, eps=1e-5, device=DEV, dtype=torch.bfloat16)
    gen = torch.Generator().manual_seed(8)
    x, g, dy = (torch.randn(2, 40, 4, 128, generator=gen).bfloat16() for _ in range(3))
    with torch.no_grad():
        norm.weight.copy_(torch.randn(128, generator=gen))
    xd, gd = x.to(DEV).requires_grad_(True), g.to(DEV).requires_grad_(True)
    outs = []
    for _ in range(2):
        y = norm(xd, gd)
        outs.append(torch.autograd.grad((y.float() * dy.to(DEV).float()).sum(), (xd, gd, norm.weight)))
    assert all(torch.equal(a, c) for a, c in zip(*outs))       # fixed summation order
    ref = M.norm_gated_grads(x.reshape(-1, 128), g.reshape(-1, 128), norm.weight.detach().cpu(), None, None, dy.reshape(-1, 128),
                             None, 1e-5, 'swish', True)
    _close('dx', ref['dx'].reshape(x.shape), outs[0][0], torch.bfloat16)
    _close('dg', ref['dg'].reshape(x.shape), outs[0][1], torch.bfloat16)
    _close('dw', ref['dw'], outs[0][2], torch.bfloat16)
    big = torch.randn(4, 4096, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    y = mods.rms_norm_gated(big, big.detach(), None, None)
    with pytest.raises(NotImplementedError, match='up to 2048'):
        y.sum().backward()


def test_modules_backward_c_entry_checks():
    from fla_hip import _lib
    lib = _lib.load()
    x = torch.zeros(1, 64, 64, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(64, 4, dtype=torch.bfloat16, device=DEV)
    dx = torch.empty_like(x)
    dwp = torch.empty(1, 64, 4, device=DEV)

    def conv(D=64, W=4, tiles=1, dw=dwp, stride=64):
        return lib.gdn_causal_conv1d_bwd(x.data_ptr(), w.data_ptr(), None, None, x.data_ptr(), None, dx.data_ptr(),
                                         None if dw is None else dw.data_ptr(), None, None, None, None,
                                         1, 64, D, W, 1, tiles, 64 * stride, stride, _lib.DTYPE_BF16, _lib.DTYPE_BF16, _lib.DTYPE_F32,
                                         _lib.ACT_SILU, 0, 0)

    assert conv() == _lib.GDN_OK
    assert conv(W=9) == _lib.GDN_ERR_UNSUPPORTED
    assert conv(tiles=2) == _lib.GDN_ERR_INVALID
    assert conv(dw=None) == _lib.GDN_ERR_INVALID
    assert conv(D=63, stride=63) == _lib.GDN_ERR_UNSUPPORTED               # channels go in pairs

    rstd = torch.ones(64, device=DEV)
    xr = torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV)
    out = torch.empty_like(xr)

    def norm(D=64, ld=64, parts=2, rs=rstd, rms=1):
        return lib.gdn_norm_gated_bwd(xr.data_ptr(), xr.data_ptr(), xr.data_ptr(), None, None, None, None if rs is None else rs.data_ptr(), None,
                                      out.data_ptr(), out.data_ptr(), None, None, 64, D, ld, parts, _lib.DTYPE_BF16, _lib.DTYPE_F32,
                                      _lib.ACT_SILU, rms, 0)

    assert norm() == _lib.GDN_OK
    assert norm(D=60) == _lib.GDN_OK                            # a row pitch above D
    assert norm(ld=60, D=60) == _lib.GDN_ERR_UNSUPPORTED
    assert norm(parts=0) == _lib.GDN_ERR_INVALID
    assert norm(rs=None) == _lib.GDN_ERR_INVALID
    assert norm(rms=0) == _lib.GDN_ERR_INVALID                  # layer norm without the means
    torch.cuda.synchronize()


@pytest.mark.parametrize('seed', range(16))
def test_conv_backward_random_configuration(seed):
    """Seeded random shapes and options: kernel sizes 1..8, odd and even channel counts, dense or packed with sequences from
    empty to several tiles long, with or without bias / residual / initial state and final-state gradient, all three dtypes."""
    gen = torch.Generator().manual_seed(2000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))
    W = r(1, 8)
    D = [2, 6, 33, 64, 130, 256, 500][r(0, 6)]
    dtype = [torch.float32, torch.float16, torch.bfloat16][r(0, 2)]
    activation = [None, 'silu'][r(0, 1)]
    has_bias, has_residual, state = bool(r(0, 1)), bool(r(0, 1)), bool(r(0, 1))
    if r(0, 1):
        lens = [[0, 1, 2, W - 1, W, 63, 64, 65, 130, 200][r(0, 9)] for _ in range(r(1, 5))]
        if sum(lens) == 0:
            lens[-1] = 3
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        case = _conv_case(1, cu[-1], D, W, dtype, has_bias, has_residual, state=state, N=len(lens), seed=seed)
        _check_conv(case, activation, cu, [torch.int32, torch.int64][r(0, 1)])
    else:
        B, T = r(1, 3), [1, 2, 7, 64, 65, 129, 300][r(0, 6)]
        _check_conv(_conv_case(B, T, D, W, dtype, has_bias, has_residual, state=state, seed=seed), activation)


@pytest.mark.parametrize('seed', range(16))
def test_norm_gated_backward_random_configuration(seed):
    gen = torch.Generator().manual_seed(3000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))
    D = [8, 50, 64, 100, 128, 256, 384, 520, 1024, 2048][r(0, 9)]
    rows = [1, 3, 40, 257, 1000][r(0, 4)]
    dtype = [torch.float32, torch.float16, torch.bfloat16][r(0, 2)]
    is_rms = bool(r(0, 1))
    affine = bool(r(0, 1))
    bias = affine and not is_rms and bool(r(0, 1))
    residual = bool(r(0, 1))
    prenorm = residual and bool(r(0, 1))
    _check_norm((rows,), D, dtype, affine, bias, ['swish', 'sigmoid'][r(0, 1)], is_rms, residual=residual, prenorm=prenorm,
                fp32_stream=prenorm and bool(r(0, 1)), seed=seed)


def test_modules_backward_without_tokens():
    """No tokens at all: zero parameter gradients, an initial state that is handed straight on to the final state."""
    mods = _mods()
    x = torch.zeros(2, 0, 64, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    w = torch.randn(64, 4, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    b = torch.randn(64, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    h0 = torch.randn(2, 64, 4, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    y, final = mods.causal_conv1d(x, w, b, None, h0, True, 'silu')
    assert y.shape == (2, 0, 64) and torch.equal(final, h0.detach())
    dht = torch.randn_like(final)
    (final.float() * dht.float()).sum().backward()
    assert torch.equal(h0.grad, dht) and not w.grad.any() and not b.grad.any() and x.grad.shape == x.shape
    xn = torch.zeros(0, 128, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    wn = torch.randn(128, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    out = mods.rms_norm_gated(xn, xn.detach(), wn, None)
    out.sum().backward()
    assert xn.grad.shape == xn.shape and not wn.grad.any()
