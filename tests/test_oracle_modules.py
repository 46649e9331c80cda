"""Pins the CPU oracle of the convolution and the gated normalisation (oracle/modules_oracle.py) without
running the reference: a library routine, a scalar loop, and invariants, each chosen so that a plausible slip
(reversed taps, state read one place off, activation after the residual, biased variance) fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import modules_oracle as M

DT = torch.float64


def _conv_inputs(B, T, D, W, seed=0, state=False, N=None):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(B, T, D, generator=gen, dtype=DT)
    w = torch.randn(D, W, generator=gen, dtype=DT)
    b = torch.randn(D, generator=gen, dtype=DT)
    r = torch.randn(B, T, D, generator=gen, dtype=DT)
    s = torch.randn(N or B, D, W, generator=gen, dtype=DT) if state else None
    return x, w, b, r, s


@pytest.mark.parametrize('W', [1, 2, 3, 4, 7])
@pytest.mark.parametrize('activation', [None, 'silu'])
def test_conv_matches_library_conv1d(W, activation):
    # the routine the reference's tests compare with (tests/modules/test_conv.py:30-72): depthwise conv1d, left padding W-1
    x, w, b, r, _ = _conv_inputs(2, 37, 6, W)
    ref = F.conv1d(x.transpose(1, 2), w[:, None, :], b, padding=W - 1, groups=6)[..., :37].transpose(1, 2)
    ref = (F.silu(ref) if activation else ref) + r
    y, _ = M.causal_conv1d(x, w, b, r, activation=activation, dtype=DT)
    assert torch.allclose(y, ref, atol=1e-12)


def test_conv_with_state_matches_library_conv1d_on_the_joined_sequence():
    # history in front of the sequence, no padding: entries 1..W-1 of the state are positions -(W-1)..-1
    W, D, T = 4, 5, 19
    x, w, b, _, s = _conv_inputs(2, T, D, W, seed=1, state=True)
    joined = torch.cat([s[:, :, 1:], x.transpose(1, 2)], dim=-1)
    ref = F.conv1d(joined, w[:, None, :], b, padding=0, groups=D).transpose(1, 2)
    y, final = M.causal_conv1d(x, w, b, initial_state=s, output_final_state=True, dtype=DT)
    assert torch.allclose(y, ref, atol=1e-12)
    assert torch.equal(final, x[:, T - W:].transpose(1, 2))
    # entry 0 of the state is never read
    s2 = s.clone(); s2[:, :, 0] += 100.0
    y2, _ = M.causal_conv1d(x, w, b, initial_state=s2, dtype=DT)
    assert torch.equal(y, y2)


def test_conv_scalar_loop():
    B, T, D, W = 2, 6, 3, 3
    x, w, b, r, s = _conv_inputs(B, T, D, W, seed=2, state=True)
    y, final = M.causal_conv1d(x, w, b, r, s, True, 'swish', dtype=DT)
    for n in range(B):
        for d in range(D):
            def at(p):                                  # input at position p of sequence n, channel d
                return x[n, p, d].item() if p >= 0 else s[n, d, W + p].item()
            for t in range(T):
                a = sum(w[d, j].item() * at(t - (W - 1) + j) for j in range(W)) + b[d].item()
                a = a / (1.0 + math.exp(-a)) + r[n, t, d].item()
                assert abs(y[n, t, d].item() - a) < 1e-12
            for j in range(W):
                assert final[n, d, j].item() == at(T - W + j)


@pytest.mark.parametrize('T', [1, 2, 3, 9])
def test_short_sequences_keep_old_state_entries(T):
    # a sequence shorter than the state leaves the newest old entries in front of its own tokens
    W, D = 4, 3
    x, w, _, _, s = _conv_inputs(1, T, D, W, seed=3, state=True)
    _, final = M.causal_conv1d(x, w, initial_state=s, output_final_state=True, dtype=DT)
    joined = torch.cat([s[0].T, x[0]], dim=0)
    assert torch.equal(final[0].T, joined[-W:])
    _, final0 = M.causal_conv1d(x, w, output_final_state=True, dtype=DT)
    joined0 = torch.cat([torch.zeros(W, D, dtype=DT), x[0]], dim=0)
    assert torch.equal(final0[0].T, joined0[-W:])


def test_split_in_time_hands_the_state_over():
    W, D, T = 4, 4, 21
    x, w, b, r, s = _conv_inputs(2, T, D, W, seed=4, state=True)
    y, final = M.causal_conv1d(x, w, b, r, s, True, 'silu', dtype=DT)
    for cut in (1, 2, 5, 20):
        y1, s1 = M.causal_conv1d(x[:, :cut], w, b, r[:, :cut], s, True, 'silu', dtype=DT)
        y2, s2 = M.causal_conv1d(x[:, cut:], w, b, r[:, cut:], s1, True, 'silu', dtype=DT)
        assert torch.allclose(torch.cat([y1, y2], 1), y, atol=1e-12)
        assert torch.equal(s2, final)


def test_updates_token_by_token_equal_one_prefill():
    W, D, T, N = 3, 5, 8, 2
    x, w, b, r, s = _conv_inputs(N, T, D, W, seed=5, state=True)
    y, final = M.causal_conv1d(x, w, b, r, s, True, 'silu', dtype=DT)
    cache = s.clone()
    for t in range(T):
        yt, cache = M.causal_conv1d_update(x[:, t], cache, w, b, r[:, t], 'silu', dtype=DT)
        assert torch.allclose(yt, y[:, t], atol=1e-12)
    assert torch.equal(cache, final)


def test_packed_equals_per_sequence():
    W, D = 4, 3
    lens = [5, 1, 0, 9, 2]
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    x, w, b, r, s = _conv_inputs(1, cu[-1], D, W, seed=6, state=True, N=len(lens))
    y, final = M.causal_conv1d(x, w, b, r, s, True, 'silu', cu_seqlens=cu, dtype=DT)
    for n in range(len(lens)):
        sl = slice(cu[n], cu[n + 1])
        yn, fn = M.causal_conv1d(x[:, sl], w, b, r[:, sl], s[n:n + 1], True, 'silu', dtype=DT)
        assert torch.equal(y[:, sl], yn)
        assert torch.equal(final[n:n + 1], fn)


@pytest.mark.parametrize('activation', ['swish', 'sigmoid'])
@pytest.mark.parametrize('is_rms', [False, True])
def test_norm_gated_matches_library_norms(activation, is_rms):
    gen = torch.Generator().manual_seed(7)
    T, D, eps = 9, 24, 1e-5
    x, g, res = (torch.randn(T, D, generator=gen, dtype=DT) for _ in range(3))
    w, b = torch.randn(D, generator=gen, dtype=DT), torch.randn(D, generator=gen, dtype=DT)
    y, r, mean, rstd = M.norm_gated(x, g, w, b, res, eps, activation, is_rms, dtype=DT)
    assert torch.equal(r, x + res)
    normed = F.rms_norm(r, (D,), w, eps) + b if is_rms else F.layer_norm(r, (D,), w, b, eps)
    gate = F.silu(g) if activation == 'swish' else torch.sigmoid(g)
    assert torch.allclose(y, normed * gate, atol=1e-12)
    var = r.var(-1, unbiased=False) if not is_rms else (r * r).mean(-1)
    assert torch.allclose(rstd, (var + eps).rsqrt(), atol=1e-12)
    assert torch.allclose(mean, torch.zeros(T, dtype=DT) if is_rms else r.mean(-1), atol=1e-14)


def test_norm_gated_special_cases():
    # constant rows: layer norm gives bias only; rms norm of a row of c gives sign(c) * weight (eps -> 0)
    T, D = 3, 8
    x = torch.full((T, D), 2.5, dtype=DT)
    g = torch.zeros(T, D, dtype=DT)                     # sigmoid(0) = 1/2
    w = torch.arange(1, D + 1, dtype=DT)
    b = torch.arange(D, dtype=DT)
    y, *_ = M.norm_gated(x, g, w, b, None, 0.0, 'sigmoid', True, dtype=DT)
    assert torch.allclose(y, (w + b).expand(T, D) * 0.5, atol=1e-12)
    y, *_ = M.norm_gated(x, g, w, b, None, 1e-5, 'sigmoid', False, dtype=DT)
    assert torch.allclose(y, b.expand(T, D) * 0.5, atol=1e-12)


# --------------------------------------------------------------------------- #
# gradients
# --------------------------------------------------------------------------- #
def _fd(fn, t, eps=1e-6):
    """Central finite differences of the scalar fn() with respect to every element of the fp64 tensor t."""
    out = torch.zeros_like(t)
    flat, oflat = t.view(-1), out.view(-1)
    for i in range(flat.numel()):
        keep = flat[i].item()
        flat[i] = keep + eps
        up = fn()
        flat[i] = keep - eps
        down = fn()
        flat[i] = keep
        oflat[i] = (up - down) / (2 * eps)
    return out


@pytest.mark.parametrize('activation', [None, 'silu'])
@pytest.mark.parametrize('packed', [False, True])
def test_conv_gradients_against_finite_differences(activation, packed):
    """Every gradient the convolution's backward returns (input, taps, bias, residual, initial state), with the gradient of
    the final state flowing in, against central differences of the forward in fp64; sequences shorter than the kernel
    hand part of the initial state on to the final state."""
    gen = torch.Generator().manual_seed(5)
    W, D = 4, 3
    if packed:
        cu, B, T = [0, 2, 2, 9], 1, 9
    else:
        cu, B, T = None, 2, 5
    N = B if cu is None else len(cu) - 1
    x, w, b, r, h0 = (torch.randn(*s, generator=gen, dtype=torch.float64) for s in ((B, T, D), (D, W), (D,), (B, T, D), (N, D, W)))
    dy = torch.randn(B, T, D, generator=gen, dtype=torch.float64)
    dht = torch.randn(N, D, W, generator=gen, dtype=torch.float64)
    grads = M.conv_grads(x, w, b, r, h0, dy, dht, activation, cu)

    def loss():
        y, final = M.causal_conv1d(x, w, b, r, h0, True, activation, cu, torch.float64)
        return ((y * dy).sum() + (final * dht).sum()).item()

    for name, t in (('dx', x), ('dw', w), ('db', b), ('dr', r), ('dh0', h0)):
        assert (grads[name] - _fd(loss, t)).abs().max() < 1e-7, name
    assert torch.equal(grads['dr'], dy)                         # the residual's gradient is dy itself
    assert (grads['dh0'][:, :, 0].abs().max() == 0) == (not packed)      # entry 0 only matters to a sequence without tokens


def test_conv_gradient_closed_forms():
    """One tap and no activation: dx = w dy, dw = sum dy x; two taps: the gradient of x[t] collects dy[t] w[1] + dy[t+1] w[0]."""
    gen = torch.Generator().manual_seed(6)
    x, dy = torch.randn(1, 6, 2, generator=gen, dtype=torch.float64), torch.randn(1, 6, 2, generator=gen, dtype=torch.float64)
    w1 = torch.randn(2, 1, generator=gen, dtype=torch.float64)
    g1 = M.conv_grads(x, w1, None, None, None, dy)
    assert torch.allclose(g1['dx'], dy * w1[:, 0]) and torch.allclose(g1['dw'][:, 0], (dy * x).sum((0, 1)))
    w2 = torch.randn(2, 2, generator=gen, dtype=torch.float64)
    g2 = M.conv_grads(x, w2, None, None, None, dy)
    want = dy * w2[:, 1]
    want[:, :-1] += dy[:, 1:] * w2[:, 0]
    assert torch.allclose(g2['dx'], want)


@pytest.mark.parametrize('activation', ['swish', 'sigmoid'])
@pytest.mark.parametrize('is_rms', [False, True])
def test_norm_gated_gradients_against_finite_differences(activation, is_rms):
    gen = torch.Generator().manual_seed(7)
    T, D = 3, 5
    x, g, r, dy, dres = (torch.randn(T, D, generator=gen, dtype=torch.float64) for _ in range(5))
    w, b = torch.randn(D, generator=gen, dtype=torch.float64), torch.randn(D, generator=gen, dtype=torch.float64)
    grads = M.norm_gated_grads(x, g, w, b, r, dy, dres, 1e-5, activation, is_rms)

    def loss():
        y, rr, _, _ = M.norm_gated(x, g, w, b, r, 1e-5, activation, is_rms, torch.float64)
        return ((y * dy).sum() + (rr * dres).sum()).item()

    for name, t in (('dx', x), ('dg', g), ('dw', w), ('db', b), ('dr', r)):
        assert (grads[name] - _fd(loss, t)).abs().max() < 1e-7, name
    assert torch.equal(grads['dx'], grads['dr'])                # x and the residual enter as their sum
