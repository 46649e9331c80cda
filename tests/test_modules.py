"""GPU parity of the convolution and the gated normalisation (through the C ABI, via fla_hip.modules) against
the CPU oracle, on the matrices of the reference's own tests (tests/modules/test_conv.py,
tests/modules/test_layernorm_gated.py).

Tolerances: the oracle is the exact fp32 formula on the rounded inputs, so what remains is the rounding of the
output to its dtype (bf16 2^-9, fp16 2^-12 relative) plus fp32 summation order: rel-RMSE <= 3e-3 (bf16),
5e-4 (fp16), 2e-6 (fp32); the reference's own tests use 1e-3.  States and caches are copies of inputs and must
be bit-exact."""
import pytest
import torch

from oracle import modules_oracle as M
from oracle.gdn_oracle import get_err_ratio

pytestmark = pytest.mark.gpu

DEV = 'cuda'
TOL = {torch.float32: 2e-6, torch.float16: 5e-4, torch.bfloat16: 3e-3}


def _mods():
    import fla_hip.modules as mods
    return mods


def _close(name, ref, tri, dtype):
    assert tri.dtype == dtype, (name, tri.dtype)
    err = get_err_ratio(ref.float(), tri.float().cpu())
    assert err <= TOL[dtype], f'{name}: rel-RMSE {err:.3e} > {TOL[dtype]:.1e}'


def _inputs(B, T, D, W, dtype, has_bias, has_residual, seed=42, N=None, state=False):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(B, T, D, generator=gen).to(dtype)
    w = torch.randn(D, W, generator=gen).to(dtype)
    b = torch.randn(D, generator=gen).to(dtype) if has_bias else None
    r = torch.randn(B, T, D, generator=gen).to(dtype) if has_residual else None
    s = torch.randn(N or B, D, W, generator=gen).to(dtype) if state else None
    return x, w, b, r, s


def _gpu(*ts):
    return [None if t is None else t.to(DEV) for t in ts]


DENSE = [
    (2, 64, 128, 3, 'swish', True, True, torch.float32),
    (2, 128, 128, 4, 'swish', False, True, torch.float32),
    (2, 64, 128, 3, 'swish', True, False, torch.float32),
    (2, 128, 128, 4, 'swish', False, False, torch.float32),
    (2, 500, 1024, 3, None, True, True, torch.float32),
    (2, 1024, 1024, 4, None, False, True, torch.float32),
    (2, 64, 128, 3, None, True, False, torch.float16),
    (2, 128, 128, 4, None, False, False, torch.float16),
    (2, 64, 100, 3, 'swish', True, True, torch.float32),       # tests/modules/test_conv.py:877
    (2, 500, 1024, 4, 'silu', True, True, torch.bfloat16),
    (3, 77, 200, 2, 'silu', False, False, torch.bfloat16),
    (1, 33, 100, 7, None, True, False, torch.bfloat16),        # channels not a multiple of 8: element-wise path
    (2, 40, 64, 1, 'silu', True, False, torch.float16),
    (2, 40, 64, 8, None, False, True, torch.float32),
]


@pytest.mark.parametrize(('B', 'T', 'D', 'W', 'activation', 'has_bias', 'has_residual', 'dtype'), DENSE)
def test_conv_dense(B, T, D, W, activation, has_bias, has_residual, dtype):
    x, w, b, r, _ = _inputs(B, T, D, W, dtype, has_bias, has_residual)
    ref, ref_state = M.causal_conv1d(x, w, b, r, None, True, activation)
    gx, gw, gb, gr = _gpu(x, w, b, r)
    for backend in ('triton', 'cuda'):
        tri, state = _mods().causal_conv1d(gx, gw, gb, residual=gr, activation=activation, backend=backend,
                                           output_final_state=True)
        _close('y', ref, tri, dtype)
        assert torch.equal(state.cpu().float(), ref_state)
    tri, none = _mods().causal_conv1d(gx, gw, gb, residual=gr, activation=activation)
    assert none is None
    _close('y', ref, tri, dtype)


VARLEN = [
    (4, 500, 128, 3, 'swish', True, True, torch.float32),
    (4, 1024, 200, 4, 'swish', False, True, torch.float32),
    (4, 500, 128, 3, None, True, False, torch.float16),
    (4, 1024, 1024, 4, None, False, False, torch.float16),
    (4, 1024, 4096, 4, 'swish', False, False, torch.bfloat16),  # tests/modules/test_conv.py:799-802 (width and length)
    (9, 700, 100, 4, 'silu', True, True, torch.bfloat16),
]


@pytest.mark.parametrize(('N', 'T', 'D', 'W', 'activation', 'has_bias', 'has_residual', 'dtype'), VARLEN)
@pytest.mark.parametrize('cu_dtype', [torch.int64, torch.int32])
def test_conv_varlen(N, T, D, W, activation, has_bias, has_residual, dtype, cu_dtype):
    torch.manual_seed(42)                                       # the reference's recipe (tests/modules/test_conv.py:225-229)
    cu = torch.cat([torch.tensor([0]), torch.arange(16, T)[torch.randperm(T - 16)[:N - 1]], torch.tensor([T])]).sort()[0]
    x, w, b, r, s = _inputs(1, T, D, W, dtype, has_bias, has_residual, N=N, state=True)
    gx, gw, gb, gr, gs = _gpu(x, w, b, r, s)
    for state in (None, s):
        ref, ref_state = M.causal_conv1d(x, w, b, r, state, True, activation, cu_seqlens=cu.tolist())
        tri, tri_state = _mods().causal_conv1d(gx, gw, gb, residual=gr, initial_state=None if state is None else gs,
                                               output_final_state=True, activation=activation,
                                               cu_seqlens=cu.to(DEV, cu_dtype))
        _close('y', ref, tri, dtype)
        assert torch.equal(tri_state.cpu().float(), ref_state)


def test_conv_varlen_with_empty_and_short_sequences_and_tokens_outside():
    # empty sequences, sequences shorter than the kernel, and a tail of tokens that belongs to no sequence
    lens = [3, 0, 1, 70, 0, 2, 33, 1]
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    T, D, W = cu[-1] + 5, 72, 4
    x, w, b, r, s = _inputs(1, T, D, W, torch.bfloat16, True, True, N=len(lens), state=True)
    ref, ref_state = M.causal_conv1d(x[:, :cu[-1]], w, b, r[:, :cu[-1]], s, True, 'silu', cu_seqlens=cu)
    gx, gw, gb, gr, gs = _gpu(x, w, b, r, s)
    tri, tri_state = _mods().causal_conv1d(gx, gw, gb, residual=gr, initial_state=gs, output_final_state=True,
                                           activation='silu', cu_seqlens=torch.tensor(cu, device=DEV))
    _close('y', ref, tri[:, :cu[-1]], torch.bfloat16)
    assert torch.equal(tri_state.cpu().float(), ref_state)


WITH_STATE = [
    (3, 128, 64, 4, 'swish', True, True, torch.float32),        # tests/modules/test_conv.py:430-435
    (4, 256, 128, 3, None, False, True, torch.float32),
    (2, 64, 128, 4, 'swish', True, False, torch.float16),
    (3, 200, 64, 3, None, False, False, torch.float16),
    (2, 3, 64, 4, 'swish', True, True, torch.float32),          # T < W
    (2, 3, 64, 3, None, False, True, torch.float32),
    (2, 1, 64, 4, 'silu', True, False, torch.bfloat16),
]


@pytest.mark.parametrize(('N', 'T', 'D', 'W', 'activation', 'has_bias', 'has_residual', 'dtype'), WITH_STATE)
def test_short_convolution_layer_prefill_with_cache(N, T, D, W, activation, has_bias, has_residual, dtype):
    # the layer on packed input with a cache, as tests/modules/test_conv.py:438-516
    mods = _mods()
    lengths = [max(1, T // N)] * N
    lengths[-1] += T % N
    T = sum(lengths)
    cu = [0]
    for n in lengths:
        cu.append(cu[-1] + n)
    x, _, _, r, s = _inputs(1, T, D, W, dtype, False, has_residual, N=N, state=True)
    torch.manual_seed(1)
    conv = mods.ShortConvolution(hidden_size=D, kernel_size=W, bias=has_bias, activation=activation, device=DEV, dtype=dtype)
    with torch.no_grad():
        conv.weight.normal_()
        if has_bias:
            conv.bias.normal_()
    w = conv.weight.detach().squeeze(1).cpu()
    b = conv.bias.detach().cpu() if has_bias else None
    s[:, :, 0] = 0
    ref, ref_state = M.causal_conv1d(x, w, b, r, s, True, activation, cu_seqlens=cu)
    gx, gr, gs = _gpu(x, r, s)
    with torch.no_grad():
        tri, cache_out = conv(gx, residual=gr, cache=gs.clone(), cu_seqlens=torch.tensor(cu, device=DEV, dtype=torch.int32),
                              output_final_state=True)
    _close('y', ref, tri, dtype)
    assert torch.equal(cache_out.cpu().float(), ref_state)
    for i in range(N):                                          # the reference's own statement of the expected cache
        for p in range(1, W):
            expected = x[0, cu[i + 1] - p] if p <= lengths[i] else s[i, :, W - (p - lengths[i])]
            assert torch.equal(cache_out[i, :, -p].cpu(), expected)


DECODE = [
    (2, 64, 128, 3, 'swish', True, True, torch.float32),        # tests/modules/test_conv.py:280-287
    (2, 128, 128, 4, 'swish', False, True, torch.float32),
    (2, 64, 128, 3, 'swish', True, False, torch.float32),
    (2, 128, 128, 4, 'swish', False, False, torch.float32),
    (2, 500, 1024, 3, None, True, True, torch.float32),
    (2, 64, 128, 3, None, True, False, torch.float16),
    (2, 128, 128, 4, None, False, False, torch.float16),
    (4, 40, 100, 4, 'silu', True, True, torch.bfloat16),
]


@pytest.mark.parametrize(('B', 'T', 'D', 'W', 'activation', 'has_bias', 'has_residual', 'dtype'), DECODE)
@pytest.mark.parametrize('layout', ['n1d', '1nd', 'nd', 'slice'])
def test_conv_decoding_token_by_token(B, T, D, W, activation, has_bias, has_residual, dtype, layout):
    T = min(T, 48)
    x, w, b, r, s = _inputs(B, T, D, W, dtype, has_bias, has_residual, state=True)
    ref, ref_state = M.causal_conv1d(x, w, b, r, s, True, activation)
    gx, gw, gb, gr, gs = _gpu(x, w, b, r, s)
    if layout == 'slice':                                       # x is a view into a wider projection (test_conv.py:720-790)
        wide = torch.randn(B, T, 3 * D, device=DEV).to(dtype)
        wide[..., D:2 * D] = gx
        gx = wide[..., D:2 * D]
    cache = gs.clone()
    tri = torch.empty(B, T, D, dtype=dtype, device=DEV)
    for t in range(T):
        xt = gx[:, t:t + 1]
        rt = gr[:, t:t + 1] if has_residual else None
        if layout == '1nd':
            xt, rt = xt.transpose(0, 1), (rt.transpose(0, 1) if rt is not None else None)
        elif layout == 'nd':
            xt, rt = xt[:, 0], (rt[:, 0] if rt is not None else None)
        y, out_cache = _mods().causal_conv1d_update(x=xt, cache=cache, residual=rt, weight=gw, bias=gb, activation=activation)
        assert out_cache is cache and y.shape == xt.shape
        tri[:, t] = y.reshape(B, D)
    _close('y', ref, tri, dtype)
    assert torch.equal(cache.cpu().float(), ref_state)


def test_layer_decodes_after_prefill():
    # prefill leaves a cache; steps through the layer continue it; together they equal one long prefill
    mods = _mods()
    B, T, D, W, dtype = 3, 50, 256, 4, torch.bfloat16
    x, _, _, _, _ = _inputs(B, T + 6, D, W, dtype, False, False)
    torch.manual_seed(2)
    conv = mods.ShortConvolution(D, W, bias=True, activation='silu', device=DEV, dtype=dtype)
    with torch.no_grad():
        conv.weight.normal_(); conv.bias.normal_()
    ref, ref_state = M.causal_conv1d(x, conv.weight.detach().squeeze(1).cpu(), conv.bias.detach().cpu(), None, None, True, 'silu')
    gx = x.to(DEV)
    with torch.no_grad():
        y0, cache = conv(gx[:, :T], output_final_state=True)
        ys = [y0]
        for t in range(T, T + 6):
            yt, cache2 = conv(gx[:, t:t + 1], cache=cache, output_final_state=True)
            assert cache2 is cache
            ys.append(yt)
    _close('y', ref, torch.cat(ys, 1), dtype)
    assert torch.equal(cache.cpu().float(), ref_state)


def test_conv_reads_a_slice_of_a_wider_projection_in_place():
    # q, k, v of the layer are column blocks of one projection; nothing is copied
    B, T, W, dtype = 2, 300, 4, torch.bfloat16
    dims = [256, 256, 512]
    gen = torch.Generator().manual_seed(3)
    qkv = torch.randn(B, T, sum(dims), generator=gen).to(dtype)
    gq = qkv.to(DEV)
    off = 0
    for D in dims:
        w = torch.randn(D, W, generator=gen).to(dtype)
        ref, ref_state = M.causal_conv1d(qkv[..., off:off + D], w, None, None, None, True, 'silu')
        tri, state = _mods().causal_conv1d(gq[..., off:off + D], w.to(DEV), activation='silu', output_final_state=True)
        assert tri.is_contiguous()
        _close('y', ref, tri, dtype)
        assert torch.equal(state.cpu().float(), ref_state)
        st = _mods().causal_conv1d_update_states(gq[..., off:off + D], W)
        assert torch.equal(st, state)
        off += D


def test_conv_full_width_prefill_spot_checks():
    # the layer's three convolutions as one: 32768 tokens x 8192 channels; windows of tokens against the oracle
    T, D, W, dtype = 32768, 8192, 4, torch.bfloat16
    gen = torch.Generator(device=DEV).manual_seed(5)
    x = torch.randn(1, T, D, generator=gen, device=DEV).to(dtype)
    w = torch.randn(D, W, generator=gen, device=DEV).to(dtype)
    b = torch.randn(D, generator=gen, device=DEV).to(dtype)
    y, state = _mods().causal_conv1d(x, w, b, activation='silu', output_final_state=True)
    for t0 in (0, 31, 4095, 20000, T - 40):
        lo = max(t0 - (W - 1), 0)
        ref, _ = M.causal_conv1d(x[:, lo:t0 + 40].cpu(), w.cpu(), b.cpu(), activation='silu')
        _close(f'y[{t0}:]', ref[:, t0 - lo:], y[:, t0:t0 + 40], dtype)
    assert torch.equal(state[0].T, x[0, T - W:])


def test_conv_many_tokens_few_channels():
    # more than 65535 * 32 tokens: the launch must not depend on the y extent of the grid
    B, T, D, W, dtype = 3, 740000, 8, 4, torch.bfloat16
    x, w, b, _, _ = _inputs(B, T, D, W, dtype, True, False)
    ref, ref_state = M.causal_conv1d(x, w, b, None, None, True, 'silu')
    tri, state = _mods().causal_conv1d(x.to(DEV), w.to(DEV), b.to(DEV), activation='silu', output_final_state=True)
    _close('y', ref, tri, dtype)
    assert torch.equal(state.cpu().float(), ref_state)


def test_conv_errors():
    mods = _mods()
    x = torch.randn(2, 8, 16, device=DEV)
    w = torch.randn(16, 4, device=DEV)
    with pytest.raises(ValueError):
        mods.causal_conv1d(x, w, backend='tilelang')
    with pytest.raises(ValueError):
        mods.causal_conv1d(x, w, cu_seqlens=torch.tensor([0, 8, 16], device=DEV))       # batch must be 1
    with pytest.raises(NotImplementedError):
        mods.causal_conv1d(x, w, activation='gelu')
    with pytest.raises(NotImplementedError):
        mods.causal_conv1d(x, torch.randn(16, 9, device=DEV))
    with pytest.raises(NotImplementedError):
        mods.causal_conv1d(x, w, cp_context=object())
    with pytest.raises(RuntimeError):
        mods.causal_conv1d(x.cpu(), w.cpu())


# ---------------------------------------------------------------------------------------------------------
# gated normalisation
# ---------------------------------------------------------------------------------------------------------
NORM = [
    (2, 2, 1, 64, False, 'silu', False),                        # tests/modules/test_layernorm_gated.py:27-30
    (2, 2, 512, 128, True, 'silu', True),
    (2, 2, 2048, 1200, True, 'sigmoid', False),
    (2, 2, 50, 50, False, 'sigmoid', False),
    (1, 3, 33, 512, True, 'swish', False),
    (1, 1, 7, 4096, True, 'swish', True),
    (1, 1, 5, 5000, True, 'sigmoid', True),
]


@pytest.mark.parametrize(('B', 'H', 'T', 'D', 'affine', 'activation', 'bias'), NORM)
@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('is_rms', [False, True])
def test_norm_gated_layers(B, H, T, D, affine, activation, bias, dtype, is_rms):
    mods = _mods()
    gen = torch.Generator().manual_seed(42)
    x = torch.randn(B, T, H, D, generator=gen).to(dtype)
    g = torch.randn(B, T, H, D, generator=gen).to(dtype)
    if is_rms:
        layer = mods.FusedRMSNormGated(D, elementwise_affine=affine, activation=activation, device=DEV, dtype=dtype)
    else:
        layer = mods.FusedLayerNormGated(D, elementwise_affine=affine, bias=bias, activation=activation, device=DEV, dtype=dtype)
    with torch.no_grad():
        if layer.weight is not None:
            layer.weight.normal_()
        if layer.bias is not None:
            layer.bias.normal_()
    w = layer.weight.detach().cpu() if layer.weight is not None else None
    b = layer.bias.detach().cpu() if layer.bias is not None else None
    ref, *_ = M.norm_gated(x.reshape(-1, D), g.reshape(-1, D), w, b, None, layer.eps, activation, is_rms)
    with torch.no_grad():
        tri = layer(x.to(DEV), g.to(DEV))
    assert tri.shape == x.shape
    _close('y', ref.reshape(x.shape), tri, dtype)


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16])
@pytest.mark.parametrize('D', [128, 1200, 50])
def test_norm_gated_residual_stream_and_statistics(dtype, D):
    mods = _mods()
    gen = torch.Generator().manual_seed(1)
    T = 300
    x, g, res = (torch.randn(T, D, generator=gen).to(dtype) for _ in range(3))
    w = torch.randn(D, generator=gen).to(dtype)
    gx, gg, gres, gw = _gpu(x, g, res, w)
    for is_rms in (False, True):
        ref, r, mean, rstd = M.norm_gated(x, g, w, None, res, 1e-6, 'swish', is_rms)
        y, tmean, trstd, rout = mods.layer_norm_gated_fwd(gx, gg, gw, None, 'swish', 1e-6, residual=gres, is_rms_norm=is_rms)
        _close('y', ref, y, dtype)
        _close('residual_out', r, rout, dtype)
        assert (tmean is None) == is_rms
        assert get_err_ratio(rstd, trstd.cpu()) < 2e-6
        if not is_rms:
            assert (mean - tmean.cpu()).abs().max() < 1e-5
        fn = mods.rms_norm_gated if is_rms else mods.layer_norm_gated
        y2, r2 = fn(gx, gg, gw, None, 'swish', residual=gres, prenorm=True, eps=1e-6)
        assert torch.equal(y2, y) and torch.equal(r2, rout)
        # residual_in_fp32 without a residual: the stream is x in fp32
        y3, r3 = fn(gx, gg, gw, None, 'swish', prenorm=True, residual_in_fp32=True, eps=1e-6)
        ref3, *_ = M.norm_gated(x, g, w, None, None, 1e-6, 'swish', is_rms)
        _close('y', ref3, y3, dtype)
        assert r3.dtype == torch.float32 and torch.equal(r3.cpu(), x.float())


def test_norm_gated_full_size_rows():
    # the layer's output norm at prefill size: 32768 tokens x 32 heads of 128 features
    mods = _mods()
    T, D, dtype = 32768 * 32, 128, torch.bfloat16
    gen = torch.Generator(device=DEV).manual_seed(9)
    x = torch.randn(T, D, generator=gen, device=DEV).to(dtype)
    g = torch.randn(T, D, generator=gen, device=DEV).to(dtype)
    w = torch.randn(D, generator=gen, device=DEV).to(dtype)
    y = mods.rms_norm_gated(x, g, w, None, 'swish', eps=1e-5)
    for t0 in (0, 12345, T - 100):
        ref, *_ = M.norm_gated(x[t0:t0 + 100].cpu(), g[t0:t0 + 100].cpu(), w.cpu(), None, None, 1e-5, 'swish', True)
        _close('y', ref, y[t0:t0 + 100], dtype)
    # rows are independent: permuting rows permutes the output
    perm = torch.randperm(4096, device=DEV)
    assert torch.equal(mods.rms_norm_gated(x[:4096][perm], g[:4096][perm], w, None, 'swish', eps=1e-5), y[:4096][perm])


def test_norm_gated_errors():
    mods = _mods()
    x = torch.randn(4, 16, device=DEV)
    with pytest.raises(ValueError):
        mods.rms_norm_gated(x, x, None, None, 'gelu')
    with pytest.raises(ValueError):
        mods.FusedRMSNormGated(16, activation='relu')
    with pytest.raises(RuntimeError):
        mods.layer_norm_gated_fwd(torch.randn(2, 40000, device=DEV), torch.randn(2, 40000, device=DEV), None, None)
    with pytest.raises(RuntimeError):
        mods.rms_norm_gated(x.cpu(), x.cpu(), None, None)


# ---------------------------------------------------------------------------------------------------------
# seeded random combinations
# ---------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize('seed', range(64))
def test_conv_random_configuration(seed):
    import random
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
    W = rnd.choice([1, 2, 3, 4, 4, 5, 8])
    D = rnd.choice([4, 8, 24, 64, 100, 128, 520, 1032])
    packed = rnd.random() < 0.5
    if packed:
        lens = [rnd.choice([0, 1, 2, 3, 8, 9, 31, 32, 33, 100]) for _ in range(rnd.choice([1, 2, 4, 7]))]
        if sum(lens) == 0:
            lens[0] = 5
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        B, T, N = 1, cu[-1], len(lens)
    else:
        B, T, cu = rnd.choice([1, 2, 3]), rnd.choice([1, 2, 7, 8, 9, 40, 257]), None
        N = B
    has_bias, has_res, has_state = rnd.random() < 0.5, rnd.random() < 0.4, rnd.random() < 0.5
    act = rnd.choice([None, 'silu', 'swish'])
    x, w, b, r, s = _inputs(B, T, D, W, dtype, has_bias, has_res, seed=seed, N=N, state=has_state)
    ref, ref_state = M.causal_conv1d(x, w, b, r, s, True, act, cu_seqlens=cu)
    gx, gw, gb, gr, gs = _gpu(x, w, b, r, s)
    if rnd.random() < 0.4:                                      # x as a column block of a wider tensor
        pad = rnd.choice([8, 3])
        wide = torch.zeros(B, T, D + 2 * pad, device=DEV, dtype=dtype)
        wide[..., pad:pad + D] = gx
        gx = wide[..., pad:pad + D]
    cu_t = None if cu is None else torch.tensor(cu, device=DEV, dtype=rnd.choice([torch.int32, torch.int64]))
    tri, state = _mods().causal_conv1d(gx, gw, gb, residual=gr, initial_state=gs, output_final_state=True, activation=act,
                                       cu_seqlens=cu_t)
    _close('y', ref, tri, dtype)
    assert torch.equal(state.cpu().float(), ref_state)


@pytest.mark.parametrize('seed', range(48))
def test_norm_gated_random_configuration(seed):
    import random
    rnd = random.Random(seed)
    dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
    T = rnd.choice([1, 3, 17, 64, 255, 1000])
    D = rnd.choice([8, 16, 50, 64, 96, 128, 256, 384, 512, 640, 1024, 2048, 3000, 4096])
    is_rms, act = rnd.random() < 0.6, rnd.choice(['swish', 'silu', 'sigmoid'])
    gen = torch.Generator().manual_seed(seed)
    x, g = torch.randn(T, D, generator=gen).to(dtype), torch.randn(T, D, generator=gen).to(dtype)
    w = torch.randn(D, generator=gen).to(rnd.choice([dtype, torch.float32])) if rnd.random() < 0.8 else None
    b = torch.randn(D, generator=gen).to(w.dtype) if w is not None and rnd.random() < 0.4 else None
    res = torch.randn(T, D, generator=gen).to(rnd.choice([dtype, torch.float32])) if rnd.random() < 0.3 else None
    eps = rnd.choice([1e-5, 1e-6])
    ref, r, mean, rstd = M.norm_gated(x, g, w, b, res, eps, act, is_rms)
    gx, gg, gw, gb, gres = _gpu(x, g, w, b, res)
    y, tmean, trstd, rout = _mods().layer_norm_gated_fwd(gx, gg, gw, gb, act, eps, residual=gres, is_rms_norm=is_rms)
    _close('y', ref, y, dtype)
    assert get_err_ratio(rstd, trstd.cpu()) < 2e-6
    if res is not None:
        _close('residual_out', r, rout, res.dtype)
    else:
        assert rout is gx or rout.data_ptr() == gx.data_ptr()


def test_modules_without_tokens_or_sequences():
    mods = _mods()
    x = torch.zeros(2, 0, 64, device=DEV, dtype=torch.bfloat16)
    w = torch.randn(64, 4, device=DEV, dtype=torch.bfloat16)
    h0 = torch.randn(2, 64, 4, device=DEV, dtype=torch.bfloat16)
    y, final = mods.causal_conv1d(x, w, None, None, h0, True, 'silu')
    assert y.shape == (2, 0, 64) and torch.equal(final, h0)
    y, cache = mods.causal_conv1d_update(torch.zeros(0, 64, device=DEV, dtype=torch.bfloat16),
                                         torch.zeros(0, 64, 4, device=DEV, dtype=torch.bfloat16), weight=w)
    assert y.shape[0] == 0 and cache.shape == (0, 64, 4)
    out = mods.rms_norm_gated(torch.zeros(0, 128, device=DEV, dtype=torch.bfloat16), torch.zeros(0, 128, device=DEV, dtype=torch.bfloat16),
                              torch.ones(128, device=DEV, dtype=torch.bfloat16), None)
    assert out.shape == (0, 128)
