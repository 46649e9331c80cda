"""The comba operator (chunk_comba through gdn_chunk_comba_fwd / gdn_chunk_comba_bwd, fused_recurrent_comba through the
token kernel, gdn_fused_recurrent_comba_fwd) on the HIP kernels against the CPU oracle.  Shapes, input recipes and bars of the reference's own tests (tests/ops/test_comba.py: chunk 22-... fp16,
normalised q, k, p, gates logsigmoid(rand) / normalizer with a share mask_p of them zeroed, o and ht within 0.005; the
recurrent entry point fp32 and fp16 within 0.002; packed sequences with a random fp16 initial state)."""
import ctypes

import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu


def _ops():
    from fla_hip.ops.comba import chunk_comba, fused_recurrent_comba
    return chunk_comba, fused_recurrent_comba


def _check(name, ref, got, ratio):
    got = got.detach().float().cpu()
    assert got.shape == ref.shape, f'{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}'
    assert not torch.isnan(got).any(), f'{name}: NaN'
    r, m = O.get_err_ratio(ref, got), O.max_abs_ratio(ref, got)
    assert r <= ratio and m <= 1e-2, f'{name}: rel-rmse {r:.3e} max-abs ratio {m:.3e}'


def _inputs(B, T, H, HV, D, dtype, normalizer=1.0, mask_p=0.0, seed=42, normalise=True, h0_std=1.0):
    gen = torch.Generator().manual_seed(seed)
    q, k, p = (torch.randn(B, T, H, D, generator=gen) for _ in range(3))
    if normalise:
        q, k, p = (F.normalize(x, p=2, dim=-1) for x in (q, k, p))
    q, k, p = q.to(dtype), k.to(dtype), p.to(dtype)
    v = torch.randn(B, T, HV, D, generator=gen).to(dtype)
    beta = torch.rand(B, T, HV, generator=gen).to(dtype).sigmoid()
    g = F.logsigmoid(torch.rand(B, T, HV, generator=gen)) / normalizer
    g = g * (torch.rand(B, T, HV, generator=gen) > mask_p)
    h0 = torch.randn(B, HV, D, D, generator=gen) * h0_std
    return q, k, v, p, g, beta, h0


def _cuda(*xs):
    return [None if x is None else x.cuda() for x in xs]


@pytest.mark.parametrize('B,T,H,D,scale,normalizer,mask_p,l2,dtype', [
    (1, 63, 1, 64, 1, 1, 0, False, torch.float16),
    (2, 1000, 3, 60, 1, 1, 0, False, torch.float16),
    (2, 1024, 3, 64, 0.1, 1, 0.5, False, torch.float16),
    (2, 1024, 4, 100, 1, 0.1, 0, False, torch.float16),
    (2, 1024, 4, 128, 0.1, 1, 0, True, torch.float16),
    (2, 1024, 4, 128, 0.1, 1, 0.5, False, torch.float16),
    (2, 1024, 4, 128, 0.1, 10, 0, False, torch.float16),
    (4, 2048, 8, 64, 0.1, 1, 0, True, torch.float16),
    (2, 1024, 4, 128, 0.1, 1, 0.5, True, torch.bfloat16),
])
def test_chunk_comba_reference_matrix(B, T, H, D, scale, normalizer, mask_p, l2, dtype):
    q, k, v, p, g, beta, h0 = _inputs(B, T, H, H, D, dtype, normalizer, mask_p, normalise=not l2)
    h0 = torch.zeros_like(h0)                                   # (the reference's chunk test starts from a zero state)
    ref_o, ref_ht = O.recurrent_comba(q, k, v, p, g, beta, scale, h0, True, use_qk_l2norm_in_kernel=l2)
    dq, dk, dv, dp, dg, db, dh = _cuda(q, k, v, p, g, beta, h0)
    o, ht = _ops()[0](dq, dk, dv, dp, dg, db, scale=scale, initial_state=dh, output_final_state=True, use_qk_l2norm_in_kernel=l2)
    assert o.dtype == dtype and ht.dtype == torch.float32
    _check('o', ref_o, o, 5e-3)
    _check('ht', ref_ht, ht, 5e-3)


@pytest.mark.parametrize('B,T,H,HV,D,l2,cu,dtype', [
    (2, 200, 2, 2, 256, False, None, torch.bfloat16),
    (1, 300, 2, 4, 192, True, None, torch.float16),
    (1, 260, 1, 2, 160, False, [0, 70, 71, 260], torch.bfloat16),
])
def test_chunk_comba_wide_keys_forward(B, T, H, HV, D, l2, cu, dtype):
    """Key head dims above 128: forward only, token by token on the recurrence kernel."""
    q, k, v, p, g, beta, h0 = _inputs(B, T, H, HV, D, dtype, normalise=not l2)
    if cu is not None:
        h0 = torch.randn(len(cu) - 1, HV, D, D, generator=torch.Generator().manual_seed(3))
    ref_o, ref_ht = O.recurrent_comba(q, k, v, p, g, beta, 0.1, h0, True, use_qk_l2norm_in_kernel=l2, cu_seqlens=cu)
    dq, dk, dv, dp, dg, db, dh = _cuda(q, k, v, p, g, beta, h0)
    cu_t = None if cu is None else torch.tensor(cu, device='cuda')
    o, ht = _ops()[0](dq, dk, dv, dp, dg, db, scale=0.1, initial_state=dh, output_final_state=True, use_qk_l2norm_in_kernel=l2,
                      cu_seqlens=cu_t)
    assert o.dtype == dtype and ht.dtype == torch.float32 and o.shape == v.shape
    _check('o', ref_o, o, 5e-3)
    _check('ht', ref_ht, ht, 5e-3)
    with pytest.raises(NotImplementedError, match='forward only'):
        _ops()[0](dq.requires_grad_(True), dk, dv, dp, dg, db, scale=0.1, cu_seqlens=cu_t)


@pytest.mark.parametrize('H,D,mask_p,cu,idx', [
    (4, 64, 0, [0, 15], torch.int32),
    (4, 64, 0, [0, 256, 500, 1000], torch.int32),
    (4, 64, 0.5, [0, 256, 500, 1000], torch.int64),
    (4, 100, 0, [0, 15, 100, 300, 1200, 2000], torch.int32),
    (2, 128, 0, [0, 64, 64, 200, 201], torch.int64),            # an empty sequence and one of a single token
])
def test_chunk_comba_packed_sequences(H, D, mask_p, cu, idx):
    T, N = cu[-1], len(cu) - 1
    q, k, v, p, g, beta, _ = _inputs(1, T, H, H, D, torch.float16, 1.0, mask_p)
    q = torch.randn(1, T, H, D, generator=torch.Generator().manual_seed(1)).half()      # (as there: q is not normalised)
    h0 = torch.randn(N, H, D, D, generator=torch.Generator().manual_seed(2)).half()
    ref_o, ref_ht = O.recurrent_comba(q, k, v, p, g, beta, None, h0, True, cu_seqlens=cu)
    dq, dk, dv, dp, dg, db, dh = _cuda(q, k, v, p, g, beta, h0)
    cu_t = torch.tensor(cu, dtype=idx, device='cuda')
    o, ht = _ops()[0](dq, dk, dv, dp, dg, db, initial_state=dh, output_final_state=True, cu_seqlens=cu_t)
    _check('o', ref_o, o, 5e-3)
    _check('ht', ref_ht, ht, 5e-3)
    # the same through a host copy of the boundaries
    o2, ht2 = _ops()[0](dq, dk, dv, dp, dg, db, initial_state=dh, output_final_state=True, cu_seqlens=cu_t,
                        cu_seqlens_cpu=torch.tensor(cu, dtype=idx))
    assert torch.equal(o, o2) and torch.equal(ht, ht2)


@pytest.mark.parametrize('B,T,H,D,scale,normalizer,dtype', [
    (1, 63, 1, 64, 1, 1, torch.float32),
    (2, 1024, 4, 60, 1, 1, torch.float32),
    (2, 1024, 8, 128, 1, 0.1, torch.float32),
    (2, 1024, 8, 128, 0.1, 1, torch.float32),
    (2, 1024, 8, 128, 1, 10, torch.float32),
    (4, 2048, 8, 64, 0.1, 1, torch.float32),
    (2, 1024, 8, 128, 1, 0.1, torch.float16),
    (2, 1024, 8, 128, 1, 10, torch.float16),
])
def test_fused_recurrent_comba_reference_matrix(B, T, H, D, scale, normalizer, dtype):
    q, k, v, p, g, beta, h0 = _inputs(B, T, H, H, D, dtype, normalizer)
    ref_o, ref_ht = O.recurrent_comba(q, k, v, p, g, beta, scale, h0, True)
    dq, dk, dv, dp, dg, db, dh = _cuda(q, k, v, p, g, beta, h0)
    keep = dh.clone()
    o, ht = _ops()[1](dq, dk, dp, dv, dg, db, scale=scale, initial_state=dh, output_final_state=True)
    assert o.dtype == dtype and ht.dtype == torch.float32 and torch.equal(dh, keep)
    _check('o', ref_o, o, 2e-3)
    _check('ht', ref_ht, ht, 2e-3)


@pytest.mark.parametrize('T,l2,dtype', [(1, False, torch.bfloat16), (1, True, torch.float32), (3, True, torch.float16)])
def test_fused_recurrent_comba_decode_kernel(T, l2, dtype):
    """1024 states of K = V = 128 and more take the whole-state decode kernel in its form with a second key: against the
    oracle, and against the general kernel (the same sequences in two calls of 512 states each)."""
    B, H, HV, D = 128, 4, 8, 128
    q, k, v, p, g, beta, h0 = _inputs(B, T, H, HV, D, dtype, normalise=not l2, seed=5)
    ref_o, ref_ht = O.recurrent_comba(q, k, v, p, g, beta, 0.1, h0, True, use_qk_l2norm_in_kernel=l2)
    dq, dk, dv, dp, dg, db, dh = _cuda(q, k, v, p, g, beta, h0)
    rec = _ops()[1]
    o, ht = rec(dq, dk, dp, dv, dg, db, scale=0.1, initial_state=dh, output_final_state=True, use_qk_l2norm_in_kernel=l2)
    _check('o', ref_o, o, 2e-3 if dtype == torch.float32 else 5e-3)
    _check('ht', ref_ht, ht, 2e-3 if dtype == torch.float32 else 5e-3)
    halves = [rec(dq[a:b], dk[a:b], dp[a:b], dv[a:b], dg[a:b], db[a:b], scale=0.1, initial_state=dh[a:b], output_final_state=True,
                  use_qk_l2norm_in_kernel=l2) for a, b in ((0, 64), (64, 128))]
    _check('o (general kernel)', torch.cat([x[0] for x in halves]).float().cpu(), o, 1e-4)
    _check('ht (general kernel)', torch.cat([x[1] for x in halves]).cpu(), ht, 1e-4)


def test_comba_options_and_reductions():
    """Defaults (p = k, beta = 1, no state), grouped value heads, value heads wider than the kernels' 128 columns, the split
    of a sequence at a chunk boundary handing the state over, and p = k with g = 0 against the delta rule operator."""
    chunk, recurrent = _ops()
    B, T, H, HV, D = 2, 300, 2, 4, 128
    q, k, v, p, g, beta, h0 = _inputs(B, T, H, HV, D, torch.bfloat16, seed=7)
    dq, dk, dv, dp, dg, db, dh = _cuda(q, k, v, p, g, beta, h0)
    ref_o, ref_ht = O.recurrent_comba(q, k, v, p, g, beta, None, h0, True)
    o, ht = chunk(dq, dk, dv, dp, dg, db, initial_state=dh, output_final_state=True)
    _check('gva o', ref_o, o, 5e-3)
    _check('gva ht', ref_ht, ht, 5e-3)
    o_r, ht_r = recurrent(dq, dk, dp, dv, dg, db, initial_state=dh, output_final_state=True)
    _check('gva o, token kernel', ref_o, o_r, 2e-3)
    _check('gva ht, token kernel', ref_ht, ht_r, 2e-3)
    # a beta per value column, fp32 inputs, the l2 norm of q, k and p in the kernel (token kernel only)
    gen = torch.Generator().manual_seed(8)
    bv = torch.rand(B, T, HV, D, generator=gen)
    q32, k32, p32 = (torch.randn(B, T, H, D, generator=gen) for _ in range(3))
    v32 = v.float()
    ref_o, ref_ht = O.recurrent_comba(q32, k32, v32, p32, g, bv, 0.5, h0, True, use_qk_l2norm_in_kernel=True)
    o_r, ht_r = recurrent(q32.cuda(), k32.cuda(), p32.cuda(), v32.cuda(), dg, bv.cuda(), scale=0.5, initial_state=dh,
                          output_final_state=True, use_qk_l2norm_in_kernel=True)
    assert o_r.dtype == torch.float32
    _check('vector beta o', ref_o, o_r, 1e-4)
    _check('vector beta ht', ref_ht, ht_r, 1e-4)

    ref_o, _ = O.recurrent_comba(q, k, v, None, g, None)
    o, none = chunk(dq, dk, dv, None, dg)
    assert none is None
    _check('defaults o', ref_o, o, 5e-3)

    o_a, ht_a = chunk(dq[:, :128], dk[:, :128], dv[:, :128], dp[:, :128], dg[:, :128], db[:, :128], initial_state=dh, output_final_state=True)
    o_b, ht_b = chunk(dq[:, 128:], dk[:, 128:], dv[:, 128:], dp[:, 128:], dg[:, 128:], db[:, 128:], initial_state=ht_a, output_final_state=True)
    o, ht = chunk(dq, dk, dv, dp, dg, db, initial_state=dh, output_final_state=True)
    assert torch.equal(torch.cat([o_a, o_b], 1), o) and torch.equal(ht_b, ht)

    gen = torch.Generator().manual_seed(9)
    v2 = torch.randn(B, T, HV, 200, generator=gen).bfloat16()
    h2 = torch.randn(B, HV, D, 200, generator=gen)
    ref_o, ref_ht = O.recurrent_comba(q, k, v2, p, g, beta, 0.2, h2, True)
    o, ht = chunk(dq, dk, v2.cuda(), dp, dg, db, scale=0.2, initial_state=h2.cuda(), output_final_state=True)
    _check('wide v o', ref_o, o, 5e-3)
    _check('wide v ht', ref_ht, ht, 5e-3)

    from fla_hip.ops.delta_rule import chunk_delta_rule
    zero = torch.zeros_like(dg)
    qh, kh, vh, bh = dq[:, :, :, :], dk, dv[:, :, :H], db[:, :, :H]
    o_c, ht_c = chunk(qh, kh, vh, None, zero[:, :, :H], bh, initial_state=dh[:, :H], output_final_state=True)
    o_d, ht_d = chunk_delta_rule(qh, kh, vh, bh, initial_state=dh[:, :H], output_final_state=True)
    _check('delta rule o', o_d.float().cpu(), o_c, 5e-3)
    _check('delta rule ht', ht_d.float().cpu(), ht_c, 5e-3)


def test_comba_validation():
    chunk, recurrent = _ops()
    q, k, v, p, g, beta, h0 = _cuda(*_inputs(2, 64, 2, 2, 64, torch.bfloat16))
    with pytest.raises(ValueError, match='batch size'):
        chunk(q, k, v, p, g, beta, cu_seqlens=torch.tensor([0, 64], device='cuda'))
    with pytest.raises(ValueError, match='number of initial states'):
        chunk(q[:1], k[:1], v[:1], p[:1], g[:1], beta[:1], initial_state=h0, cu_seqlens=torch.tensor([0, 64], device='cuda'))
    with pytest.raises(ValueError, match='share one shape'):
        chunk(q, k, v, p[..., :32], g, beta)
    with pytest.raises(ValueError, match='g and beta'):
        chunk(q, k, v, p, g[..., :1], beta)
    with pytest.raises(NotImplementedError, match='no backward'):
        recurrent(q.clone().requires_grad_(), k, p, v, g, beta)
    with pytest.raises(ValueError, match='beta'):
        recurrent(q, k, p, v, g, beta[..., None].expand(-1, -1, -1, 32))
    with pytest.raises(RuntimeError, match='ROCm GPU'):
        chunk(*(x.cpu() for x in (q, k, v, p, g, beta)))
    big = torch.zeros(1, 64, 1, 264, dtype=torch.bfloat16, device='cuda')
    with pytest.raises(NotImplementedError, match='key head dims'):
        chunk(big, big, big, big, g[:1, :, :1], beta[:1, :, :1])
    # no tokens: the state passes through
    e = [x[:, :0] for x in (q, k, v, p, g, beta)]
    o, ht = chunk(*e, initial_state=h0, output_final_state=True)
    assert o.shape == (2, 0, 2, 64) and torch.equal(ht, h0)


def test_comba_c_entry_checks():
    from fla_hip import _lib
    lib = _lib.load()
    x = torch.zeros(1, 64, 1, 128, dtype=torch.bfloat16, device='cuda')
    s = torch.zeros(1, 64, 1, device='cuda')
    o = torch.empty_like(x)
    ws = torch.empty(lib.gdn_chunk_kda_workspace_bytes(1, 1), dtype=torch.uint8, device='cuda')

    def call(K=128, V=128, flags=0, ws_bytes=None, p=x, num_chunks=1, qkv=_lib.DTYPE_BF16):
        return lib.gdn_chunk_comba_fwd(
            x.data_ptr(), x.data_ptr(), x.data_ptr(), None if p is None else p.data_ptr(), s.data_ptr(), s.data_ptr(), None, None, o.data_ptr(),
            None, None, None, ws.data_ptr(), ws.numel() if ws_bytes is None else ws_bytes,
            1, 64, 1, 1, K, V, 1, num_chunks, 1.0, qkv, _lib.DTYPE_F32, flags, 0)

    assert call() == _lib.GDN_OK
    assert call(K=64) == _lib.GDN_ERR_UNSUPPORTED
    assert call(flags=_lib.FLAG_BETA_SIGMOID) == _lib.GDN_ERR_UNSUPPORTED
    assert call(ws_bytes=16) == _lib.GDN_ERR_WORKSPACE
    assert call(p=None) == _lib.GDN_ERR_INVALID
    assert call(num_chunks=2) == _lib.GDN_ERR_INVALID
    assert call(qkv=_lib.DTYPE_F32) == _lib.GDN_ERR_UNSUPPORTED
    torch.cuda.synchronize()


@pytest.mark.parametrize('seed', range(12))
def test_chunk_comba_random_combinations(seed):
    """Seeded random shapes and options (lengths off the chunk grid, packed or padded batches, grouped heads, narrow head
    dims, l2 norm in the kernel, extreme and masked gates, either 16-bit type) against the oracle."""
    gen = torch.Generator().manual_seed(1000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))
    H = r(1, 3); HV = H * r(1, 2); D = [32, 60, 64, 100, 128][r(0, 4)]
    dtype = [torch.bfloat16, torch.float16][r(0, 1)]
    l2 = bool(r(0, 1)); packed = bool(r(0, 1))
    normalizer = [0.1, 1.0, 10.0][r(0, 2)]; mask_p = [0.0, 0.5][r(0, 1)]
    if packed:
        lens = [r(0, 200) for _ in range(r(1, 4))]
        if sum(lens) == 0:
            lens[0] = 5
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        B, T, N = 1, cu[-1], len(lens)
    else:
        B, T, cu = r(1, 3), r(1, 260), None
        N = B
    q, k, v, p, g, beta, _ = _inputs(B, T, H, HV, D, dtype, normalizer, mask_p, seed=seed, normalise=not l2)
    h0 = torch.randn(N, HV, D, D, generator=gen) if r(0, 1) else None
    scale = [None, 0.1, 1.0][r(0, 2)]
    ref_o, ref_ht = O.recurrent_comba(q, k, v, p, g, beta, scale, h0, True, cu_seqlens=cu, use_qk_l2norm_in_kernel=l2)
    dq, dk, dv, dp, dg, db, dh = _cuda(q, k, v, p, g, beta, h0)
    o, ht = _ops()[0](dq, dk, dv, dp, dg, db, scale=scale, initial_state=dh, output_final_state=True, use_qk_l2norm_in_kernel=l2,
                      cu_seqlens=None if cu is None else torch.tensor(cu, device='cuda'))
    _check('o', ref_o, o, 5e-3)
    _check('ht', ref_ht, ht, 5e-3)


# --------------------------------------------------------------------------------------------
# backward of chunk_comba (gdn_chunk_comba_bwd) against the oracle's gradients
# --------------------------------------------------------------------------------------------
# (tests/ops/test_comba.py:198-206 and :290-297 of the reference)
GRAD_TOL = dict(dq=0.005, dk=0.008, dv=0.005, dp=0.008, dg=0.02, dbeta=0.005, dh0=0.008)
GRAD_TOL_PACKED = dict(dq=0.007, dk=0.008, dv=0.007, dp=0.008, dg=0.015, dbeta=0.015, dh0=0.007)


def _comba_grads_gpu(q, k, v, p, g, beta, h0, do, dht, scale, cu=None, l2=False, idx_dtype=torch.int64):
    chunk_comba, _ = _ops()
    leaves = {n: (None if x is None else x.cuda().requires_grad_(True))
              for n, x in dict(dq=q, dk=k, dv=v, dp=p, dg=g, dbeta=beta, dh0=h0).items()}
    cu_t = None if cu is None else torch.tensor(cu, dtype=idx_dtype, device='cuda')
    o, ht = chunk_comba(leaves['dq'], leaves['dk'], leaves['dv'], leaves['dp'], leaves['dg'], leaves['dbeta'], scale=scale,
                        initial_state=leaves['dh0'], output_final_state=True, use_qk_l2norm_in_kernel=l2, cu_seqlens=cu_t)
    ((o.float() * do.cuda().float()).sum() + (ht * dht.cuda()).sum()).backward()
    return o, ht, {n: (None if x is None else x.grad) for n, x in leaves.items()}


def _compare_grads(ref, got, tol):
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


@pytest.mark.parametrize('B,T,H,HV,D,scale,normalizer,mask_p,l2,dtype', [
    (1, 63, 1, 1, 64, 1, 1, 0, False, torch.float16),               # the reference's matrix (shorter where it is long)
    (2, 500, 3, 3, 60, 1, 1, 0, False, torch.float16),
    (2, 300, 3, 3, 64, 0.1, 1, 0.5, False, torch.float16),
    (2, 256, 4, 4, 100, 1, 0.1, 0, False, torch.float16),
    (2, 512, 4, 4, 128, 0.1, 1, 0, True, torch.float16),
    (2, 256, 4, 4, 128, 0.1, 1, 0.5, False, torch.float16),
    (2, 256, 4, 4, 128, 0.1, 10, 0, False, torch.float16),
    (2, 200, 8, 8, 64, 0.1, 1, 0, True, torch.float16),
    (2, 200, 2, 4, 128, None, 4.0, 0, False, torch.bfloat16),       # grouped value heads
    (1, 130, 2, 6, 128, None, 4.0, 0, True, torch.bfloat16),
    (3, 100, 12, 24, 128, None, 4.0, 0, False, torch.bfloat16),     # 72 runs: the scans take 64 value columns per workgroup
    (2, 70, 80, 80, 128, None, 4.0, 0, False, torch.bfloat16),      # 160 runs: all 128
])
def test_chunk_comba_backward(B, T, H, HV, D, scale, normalizer, mask_p, l2, dtype):
    q, k, v, p, g, beta, h0 = _inputs(B, T, H, HV, D, dtype, normalizer, mask_p, normalise=not l2, h0_std=0.5)
    gen = torch.Generator().manual_seed(43)
    do = torch.randn(B, T, HV, D, generator=gen).to(dtype)
    dht = torch.randn(B, HV, D, D, generator=gen)
    ref = O.comba_grads(q, k, v, p, g, beta, do, dht, scale=scale, initial_state=h0, use_qk_l2norm_in_kernel=l2, dtype=torch.float32)
    o, ht, got = _comba_grads_gpu(q, k, v, p, g, beta, h0, do, dht, scale, l2=l2)
    ref_o, ref_ht = O.recurrent_comba(q, k, v, p, g, beta, scale, h0, True, use_qk_l2norm_in_kernel=l2)
    _check('o', ref_o, o, 0.005)
    _check('ht', ref_ht, ht, 0.005)
    _compare_grads(ref, got, GRAD_TOL)
    for n, x in dict(dq=q, dk=k, dv=v, dp=p, dg=g, dbeta=beta, dh0=h0).items():
        assert got[n].dtype == x.dtype and got[n].shape == x.shape, n


@pytest.mark.parametrize('H,D,mask_p,cu,idx_dtype', [
    (4, 64, 0, [0, 15], torch.int32),
    (4, 64, 0, [0, 256, 500, 1000], torch.int32),
    (4, 64, 0.5, [0, 256, 500, 1000], torch.int64),
    (4, 100, 0, [0, 15, 100, 300, 1200, 2000], torch.int32),
    (2, 128, 0, [0, 64, 64, 129, 400], torch.int64),                # an empty sequence, a chunk boundary
])
def test_chunk_comba_backward_packed(H, D, mask_p, cu, idx_dtype):
    T, N = cu[-1], len(cu) - 1
    q, k, v, p, g, beta, _ = _inputs(1, T, H, H, D, torch.float16, 1.0, mask_p)
    gen = torch.Generator().manual_seed(44)
    h0 = torch.randn(N, H, D, D, generator=gen)
    do = torch.randn(1, T, H, D, generator=gen).half()
    dht = torch.rand(N, H, D, D, generator=gen)
    ref = O.comba_grads(q, k, v, p, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, dtype=torch.float32)
    _, _, got = _comba_grads_gpu(q, k, v, p, g, beta, h0, do, dht, None, cu=cu, idx_dtype=idx_dtype)
    _compare_grads(ref, got, GRAD_TOL_PACKED)


def test_chunk_comba_backward_wide_values_and_outside_tokens():
    """V = 256 (two heads of 128 columns inside), and a packed tensor whose sequences leave tokens out at both ends:
    those get zero gradients."""
    B, T, H, K, V = 1, 200, 2, 64, 256
    gen = torch.Generator().manual_seed(45)
    q, k, p = (F.normalize(torch.randn(B, T, H, K, generator=gen), dim=-1).bfloat16() for _ in range(3))
    v = torch.randn(B, T, H, V, generator=gen).bfloat16()
    g = F.logsigmoid(torch.rand(B, T, H, generator=gen))
    beta = torch.rand(B, T, H, generator=gen).sigmoid()
    cu = [10, 90, 180]
    h0 = torch.randn(2, H, K, V, generator=gen) * 0.5
    do = torch.randn(B, T, H, V, generator=gen).bfloat16()
    dht = torch.randn(2, H, K, V, generator=gen)
    sl = slice(cu[0], cu[-1])
    ref = O.comba_grads(q[:, sl], k[:, sl], v[:, sl], p[:, sl], g[:, sl], beta[:, sl], do[:, sl], dht, initial_state=h0,
                        cu_seqlens=[c - cu[0] for c in cu], dtype=torch.float32)
    _, _, got = _comba_grads_gpu(q, k, v, p, g, beta, h0, do, dht, None, cu=cu)
    for n in ('dq', 'dk', 'dv', 'dp', 'dg', 'dbeta'):
        x = got[n]
        assert not x[:, :cu[0]].any() and not x[:, cu[-1]:].any(), f'{n}: tokens outside every sequence must get zero'
        got[n] = x[:, sl]
    _compare_grads(ref, got, GRAD_TOL)



@pytest.mark.parametrize('B,T,H,K,cu', [(2, 200, 3, 128, None), (1, 333, 2, 100, [0, 1, 130, 333])])
def test_chunk_comba_backward_l2norm_inside_the_kernels(B, T, H, K, cu):
    """One value head per q/k head: the l2 normalisation of q, k and p, forward and back, is taken inside the backward's
    kernels (C entry gdn_chunk_comba_bwd_qk_l2norm): against the separate route (gdn_l2norm_fwd, gdn_chunk_comba_bwd, then
    gdn_l2norm_bwd on its rounded output) and against the oracle's gradients of the rows before normalisation."""
    from fla_hip.ops.comba import chunk as M
    gen = torch.Generator().manual_seed(6)
    N = B if cu is None else len(cu) - 1
    q, k, p = (torch.randn(B, T, H, K, generator=gen).bfloat16() for _ in range(3))
    v, do = (torch.randn(B, T, H, 128, generator=gen).bfloat16() for _ in range(2))
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen)) / 2
    beta = torch.rand(B, T, H, generator=gen)
    h0, dht = 0.5 * torch.randn(N, H, K, 128, generator=gen), torch.randn(N, H, K, 128, generator=gen)
    ref = O.comba_grads(q, k, v, p, g, beta, do, dht, initial_state=h0, cu_seqlens=cu, use_qk_l2norm_in_kernel=True, dtype=torch.float32)
    cu_t = None if cu is None else torch.tensor(cu, device='cuda')
    rest = (g.cuda(), beta.cuda(), K ** -0.5, h0.cuda(), do.cuda(), dht.cuda(), cu_t, None)
    inside = M.chunk_comba_bwd(q.cuda(), k.cuda(), v.cuda(), p.cuda(), *rest, qk_l2norm=True)
    (qn, q_rstd), (kn, k_rstd), (pn, p_rstd) = (M.l2norm_fwd(x.cuda()) for x in (q, k, p))
    apart = M.chunk_comba_bwd(qn[..., :K], kn[..., :K], v.cuda(), pn[..., :K], *rest, q_rstd, k_rstd, p_rstd)
    for i, name in ((0, 'dq'), (1, 'dk'), (3, 'dp')):
        a, b = inside[i], apart[i]
        assert a.shape == b.shape == (B, T, H, K)
        r = O.get_err_ratio(b.float().cpu(), a.float().cpu())
        assert r < 5e-3, f'{name}: inside the kernels against the separate route {r:.3e}'
        e = O.get_err_ratio(ref[name], a.float().cpu())
        assert e <= GRAD_TOL[name], f'{name}: rel-rmse {e:.3e} against the oracle'
    for i, name in ((2, 'dv'), (4, 'dbeta'), (5, 'dg'), (6, 'dh0')):      # (the normalised rows may differ in their last bit)
        r = O.get_err_ratio(apart[i].float().cpu(), inside[i].float().cpu())
        assert r < 2e-3, f'{name}: {r:.3e}'
    from fla_hip import _lib
    lib = _lib.load()
    assert lib.gdn_chunk_comba_bwd_qk_l2norm_workspace_bytes(1, 2, 64) > lib.gdn_chunk_bwd_qk_l2norm_workspace_bytes(1, 2, 128, 64)
    x = torch.zeros(1, 64, 2, 128, dtype=torch.bfloat16, device='cuda')
    x1 = torch.zeros(1, 64, 1, 128, dtype=torch.bfloat16, device='cuda')
    f = torch.zeros(1, 64, 2, device='cuda')
    ws = torch.zeros(lib.gdn_chunk_comba_bwd_qk_l2norm_workspace_bytes(1, 2, 64), dtype=torch.uint8, device='cuda')
    tail = [x.data_ptr(), f.data_ptr(), f.data_ptr(), None, x.data_ptr(), None] + [x.data_ptr()] * 4 + [f.data_ptr()] * 2 + [None]
    dims = lambda h: (None, None, None, ws.data_ptr(), ws.numel(), 1, 64, h, 2, 128, 128, 1, 1, 1.0, _lib.DTYPE_BF16, _lib.DTYPE_F32, 0, None)
    rc = lib.gdn_chunk_comba_bwd_qk_l2norm(x1.data_ptr(), x1.data_ptr(), x1.data_ptr(), *tail, *dims(1))
    assert rc == _lib.GDN_ERR_UNSUPPORTED and 'H == HV' in _lib.last_error()
    assert lib.gdn_chunk_comba_bwd_qk_l2norm(x.data_ptr(), x.data_ptr(), x.data_ptr(), *tail, *dims(2)) == _lib.GDN_OK
    torch.cuda.synchronize()
