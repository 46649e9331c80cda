"""gdn_chunk_fwd_static, the entry point that allocates nothing (its workspace is a fixed array inside the
library), against gdn_chunk_fwd on the same inputs through the C ABI: bit for bit, on calls in a row that
share the array, the second with a smaller input."""
import pytest
import torch

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu


def _launch(B, T, H, HV, D, seed, cu=None, flags_env=None, V=None, **kw):
    from fla_hip.ops.gated_delta_rule.chunk import ChunkLaunch
    dev = 'cuda'
    N = B if cu is None else len(cu) - 1
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, D, V or D, seed=seed, gate_div=8.0, h0_std=0.5, N=N, dtype=torch.bfloat16)
    cu_t = None if cu is None else torch.tensor(cu, device=dev)
    return ChunkLaunch(q.to(dev), k.to(dev), v.to(dev), g.to(dev), beta.to(dev), D ** -0.5, h0.to(dev), True,
                       cu_seqlens=cu_t, **kw)


def _run_both(call):
    """Returns (o, ht) of gdn_chunk_fwd and of gdn_chunk_fwd_static for one prepared call."""
    from fla_hip import _lib
    from fla_hip.ops.gated_delta_rule._common import current_stream_ptr
    lib = _lib.load()
    stream = current_stream_ptr(call.device)
    call.o.fill_(float('nan')); call.ht.fill_(float('nan'))
    _lib.check(lib.gdn_chunk_fwd(*call.args, stream))
    torch.cuda.synchronize()
    ref = (call.o.clone(), call.ht.clone())
    call.o.fill_(float('nan')); call.ht.fill_(float('nan'))
    args = call.args[:13] + call.args[15:]                   # the same arguments without workspace and size
    _lib.check(lib.gdn_chunk_fwd_static(*args, stream))
    torch.cuda.synchronize()
    return ref, (call.o.clone(), call.ht.clone())


def test_static_workspace_entry_equals_the_allocating_one():
    from fla_hip import _lib
    from fla_hip.ops.gated_delta_rule._common import current_stream_ptr
    # a dense call that is cut into time segments, then a smaller packed one, then the first again, then wide keys
    big = _launch(1, 4096, 2, 4, 128, seed=1)
    small = _launch(1, 700, 2, 4, 128, seed=2, cu=[0, 130, 131, 500, 700])
    wide = _launch(1, 600, 2, 2, 256, seed=5, V=128)
    lib, stream = _lib.load(), current_stream_ptr(big.device)
    for name, call in (('first', big), ('second, smaller', small), ('first again', big), ('wide keys', wide)):
        ref, got = _run_both(call)
        assert not torch.isnan(got[0]).any() and not torch.isnan(got[1]).any(), name
        assert torch.equal(ref[0], got[0]) and torch.equal(ref[1], got[1]), name
    # The static entry leaves the device's free memory as it is (hipMemGetInfo).  Taken around static calls alone, after
    # every kernel they launch has run once above: the first launch of a kernel makes the runtime load its code.
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for call in (big, small, wide, big):
        _lib.check(lib.gdn_chunk_fwd_static(*(call.args[:13] + call.args[15:]), stream))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    # and it is right, not just equal
    ref, got = _run_both(big)
    q, k, v, g, beta, h0 = O.make_inputs(1, 4096, 2, 4, 128, 128, seed=1, gate_div=8.0, h0_std=0.5, dtype=torch.bfloat16)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    assert O.get_err_ratio(ref_o, got[0].float().cpu()) < 5e-3 and O.get_err_ratio(ref_ht, got[1].cpu()) < 5e-3
    assert _lib.CHUNK_STATIC_WORKSPACE_BYTES == 64 << 20


def test_static_workspace_limits():
    from fla_hip import _lib
    from fla_hip.ops.gated_delta_rule._common import current_stream_ptr
    lib = _lib.load()
    # the plan with segments does not fit (3 * 8 * 32 matrices of 64 KB), whole sequences do: same as SCAN_WIDE
    call = _launch(1, 4096, 16, 32, 128, seed=3)
    assert lib.gdn_chunk_workspace_bytes(1, 4096, 64, 16, 32, 128, 128, 0, 0) > _lib.CHUNK_STATIC_WORKSPACE_BYTES
    stream = current_stream_ptr(call.device)
    args = list(call.args)
    _lib.check(lib.gdn_chunk_fwd_static(*(args[:13] + args[15:]), stream))
    torch.cuda.synchronize()
    got = (call.o.clone(), call.ht.clone())
    args[-1] |= _lib.FLAG_SCAN_WIDE
    call.o.zero_(); call.ht.zero_()
    _lib.check(lib.gdn_chunk_fwd(*args, stream))
    torch.cuda.synchronize()
    assert torch.equal(call.o, got[0]) and torch.equal(call.ht, got[1])
    # too many records for the array: refused with a clear message, nothing launched
    huge = _launch(1, 16384, 16, 32, 128, seed=4)
    huge.o.zero_()
    rc = lib.gdn_chunk_fwd_static(*(huge.args[:13] + huge.args[15:]), stream)
    assert rc == _lib.GDN_ERR_WORKSPACE and 'built-in' in _lib.last_error()
    torch.cuda.synchronize()
    assert not huge.o.any()
