"""The Gated DeltaNet layer (fla_hip.layers.GatedDeltaNet, the reference's fla/layers/gated_deltanet.py:28-364) on
the GPU against the composition of the CPU oracles, and its cache hand-over from prefill to decode."""
import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O
from oracle import modules_oracle as M

pytestmark = pytest.mark.gpu
DEV = 'cuda'
BF = torch.bfloat16


def _layer(seed=0, **kw):
    from fla_hip.layers import GatedDeltaNet
    torch.manual_seed(seed)
    args = dict(hidden_size=256, expand_v=2, head_dim=64, num_heads=2, num_v_heads=4, layer_idx=0, conv_bias=True)
    args.update(kw)
    layer = GatedDeltaNet(**args)
    with torch.no_grad():
        for name, prm in layer.named_parameters():
            if 'conv1d' in name:
                prm.normal_(0, 0.5)
            if name == 'o_norm.weight':
                prm.normal_(1, 0.2)
    return layer.to(DEV).to(BF).eval()


def _r(x):                                                       # the rounding every stage's output goes through
    return x.to(BF).float()


def _oracle_forward(layer, x, cu=None):
    """x [B, T, hidden] (bf16 values); every stage in fp32 on the CPU, rounded to bf16 where the layer's tensors are."""
    p = {k: v.detach().float().cpu() for k, v in layer.state_dict().items()}
    x = x.float().cpu()
    lin = lambda name: _r(F.linear(x, p[f'{name}.weight']))
    q, k, v = lin('q_proj'), lin('k_proj'), lin('v_proj')
    conv = lambda t, name: _r(M.causal_conv1d(t, p[f'{name}.weight'].squeeze(1), p.get(f'{name}.bias'), activation='silu',
                                              cu_seqlens=cu)[0])
    q, k, v = conv(q, 'q_conv1d'), conv(k, 'k_conv1d'), conv(v, 'v_conv1d')
    H, HV, K, V = layer.num_heads, layer.num_v_heads, layer.head_k_dim, layer.head_v_dim
    q, k, v = q.unflatten(-1, (H, K)), k.unflatten(-1, (H, K)), v.unflatten(-1, (HV, V))
    g = O.gdn_gate(lin('a_proj'), p['A_log'], p['dt_bias'])
    beta = torch.sigmoid(lin('b_proj')) * (2.0 if layer.allow_neg_eigval else 1.0)
    o, ht = O.chunk_gated_delta_rule(O.l2norm(q), O.l2norm(k), v, g, beta, None, None, True, cu_seqlens=cu)
    o = _r(o)
    gate = lin('g_proj').unflatten(-1, (HV, V))
    y, *_ = M.norm_gated(o.reshape(-1, V), gate.reshape(-1, V), p['o_norm.weight'], None, None, layer.o_norm.eps, 'swish', True)
    y = _r(y).reshape(*o.shape[:2], HV * V)
    return F.linear(y, p['o_proj.weight']), ht


def test_parameter_names_are_the_references():
    names = {n for n, _ in _layer().named_parameters()}
    assert names == {'A_log', 'dt_bias', 'q_proj.weight', 'k_proj.weight', 'v_proj.weight', 'a_proj.weight', 'b_proj.weight',
                     'q_conv1d.weight', 'q_conv1d.bias', 'k_conv1d.weight', 'k_conv1d.bias', 'v_conv1d.weight', 'v_conv1d.bias',
                     'g_proj.weight', 'o_norm.weight', 'o_proj.weight'}


@pytest.mark.parametrize('T', [200, 40])                         # chunk kernels / token recurrence
@pytest.mark.parametrize('neg', [False, True])
def test_layer_matches_the_oracles_stage_by_stage(T, neg):
    from fla_hip.layers import LayerCache
    layer = _layer(allow_neg_eigval=neg)
    x = torch.randn(2, T, 256, generator=torch.Generator().manual_seed(1)).to(BF)
    ref, ref_state = _oracle_forward(layer, x)
    cache = LayerCache()
    out, _, cache2 = layer(x.to(DEV), past_key_values=cache, use_cache=True)
    assert cache2 is cache and len(cache) == 1 and cache.get_seq_length() == T
    assert O.get_err_ratio(ref, out.float().cpu()) < 1e-2
    st = cache[0]['recurrent_state']                             # [N, HV, V, K]: state_v_first
    assert st.dtype == torch.float32 and st.shape == (2, 4, 128, 64)
    assert O.get_err_ratio(ref_state, st.transpose(-1, -2).cpu()) < 1e-2
    for c, name in zip(cache[0]['conv_state'], ('q_proj', 'k_proj', 'v_proj')):
        want = F.linear(x.float(), getattr(layer, name).weight.float().cpu())[:, -4:].transpose(1, 2)
        assert O.get_err_ratio(want, c.float().cpu()) < 1e-2     # the last 4 inputs of each convolution
    out2, _, none = layer(x.to(DEV))                             # without a cache: same output
    assert none is None and torch.equal(out2, out)


def test_prefill_then_decode_equals_one_prefill():
    from fla_hip.layers import LayerCache
    layer = _layer(seed=3)
    T, n = 150, 6
    x = torch.randn(2, T + n, 256, generator=torch.Generator().manual_seed(2)).to(BF).to(DEV)
    whole, _, _ = layer(x)
    cache = LayerCache()
    first, _, _ = layer(x[:, :T], past_key_values=cache, use_cache=True)
    steps = [layer(x[:, T + i:T + i + 1], past_key_values=cache, use_cache=True)[0] for i in range(n)]
    assert cache.get_seq_length() == T + n
    got = torch.cat([first] + steps, 1)
    assert O.get_err_ratio(whole.float().cpu(), got.float().cpu()) < 1e-2
    ref, _ = _oracle_forward(layer, x)
    assert O.get_err_ratio(ref, got.float().cpu()) < 1e-2


def test_padding_mask_equals_each_sequence_alone():
    layer = _layer(seed=4)
    lens = [90, 37, 128]
    T = max(lens)
    x = torch.randn(3, T, 256, generator=torch.Generator().manual_seed(5)).to(BF).to(DEV)
    mask = torch.zeros(3, T, dtype=torch.long, device=DEV)
    for b, n in enumerate(lens):
        mask[b, T - n:] = 1                                      # left padding
    out, _, _ = layer(x, attention_mask=mask)
    for b, n in enumerate(lens):
        alone, _, _ = layer(x[b:b + 1, T - n:])
        assert O.get_err_ratio(alone.float().cpu(), out[b:b + 1, T - n:].float().cpu()) < 5e-3
        assert not out[b, :T - n].any()
    # explicit cu_seqlens on packed input: the same tokens
    packed = torch.cat([x[b, T - n:] for b, n in enumerate(lens)])[None]
    cu = torch.tensor([0, 90, 127, 255], device=DEV, dtype=torch.int32)
    out_p, _, _ = layer(packed, cu_seqlens=cu)
    want = torch.cat([out[b, T - n:] for b, n in enumerate(lens)])[None]
    assert torch.equal(out_p, want)


def _oracle_loss(layer, x, dy, cu=None):
    """The layer as a composition of the oracles in fp64 on the CPU, differentiable: returns the gradients of
    sum(out * dy) with respect to the input and every parameter (by name)."""
    DT = torch.float64
    p = {k: v.detach().to(DT).cpu().requires_grad_(True) for k, v in layer.state_dict().items()}
    xs = x.detach().to(DT).cpu().requires_grad_(True)
    lin = lambda name: F.linear(xs, p[f'{name}.weight'])
    conv = lambda t, name: M.causal_conv1d(t, p[f'{name}.weight'].squeeze(1), p.get(f'{name}.bias'), activation='silu',
                                           cu_seqlens=cu, dtype=DT)[0]
    q, k, v = conv(lin('q_proj'), 'q_conv1d'), conv(lin('k_proj'), 'k_conv1d'), conv(lin('v_proj'), 'v_conv1d')
    H, HV, K, V = layer.num_heads, layer.num_v_heads, layer.head_k_dim, layer.head_v_dim
    q, k, v = q.unflatten(-1, (H, K)), k.unflatten(-1, (H, K)), v.unflatten(-1, (HV, V))
    g = O.gdn_gate(lin('a_proj'), p['A_log'], p['dt_bias'])
    beta = torch.sigmoid(lin('b_proj')) * (2.0 if layer.allow_neg_eigval else 1.0)
    o, _ = O.recurrent_gated_delta_rule(O.l2norm(q), O.l2norm(k), v, g, beta, None, None, False, cu_seqlens=cu, dtype=DT)
    gate = lin('g_proj').unflatten(-1, (HV, V))
    y, *_ = M.norm_gated(o.reshape(-1, V), gate.reshape(-1, V), p['o_norm.weight'], None, None, layer.o_norm.eps, 'swish', True, DT)
    out = F.linear(y.reshape(*o.shape[:2], HV * V), p['o_proj.weight'])
    (out * dy.to(DT).cpu()).sum().backward()
    return out.detach(), xs.grad, {k: v.grad for k, v in p.items()}


@pytest.mark.parametrize('packed', [False, True])
def test_layer_trains(packed):
    """Training mode: the gradient of every parameter and of the input through the convolutions' , the chunked operator's and
    the gated norm's backward kernels against reverse-mode differentiation of the oracles' composition.  Everything between
    the projections is bf16 on the GPU, so the bar is that of a bf16 pipeline (2e-2 rel-RMSE; gate parameters, whose
    gradients are small sums of many terms, 4e-2)."""
    layer = _layer(seed=6).train()
    gen = torch.Generator().manual_seed(7)
    if packed:
        x = torch.randn(1, 230, 256, generator=gen).to(BF)
        cu = [0, 70, 71, 230]
        kw = dict(cu_seqlens=torch.tensor(cu, device=DEV, dtype=torch.int32))
    else:
        x = torch.randn(2, 150, 256, generator=gen).to(BF)
        cu, kw = None, {}
    dy = torch.randn(*x.shape[:2], 256, generator=gen).to(BF)
    xd = x.to(DEV).requires_grad_(True)
    out, _, _ = layer(xd, **kw)
    out.backward(dy.to(DEV))
    ref_out, ref_dx, ref = _oracle_loss(layer, x, dy, cu)
    assert O.get_err_ratio(ref_out, out.detach().double().cpu()) < 1e-2
    assert O.get_err_ratio(ref_dx, xd.grad.double().cpu()) < 2e-2
    for name, prm in layer.named_parameters():
        assert prm.grad is not None, name
        bar = 4e-2 if name in ('A_log', 'dt_bias') else 2e-2
        err = O.get_err_ratio(ref[name], prm.grad.double().cpu())
        assert err < bar, f'{name}: rel-RMSE {err:.3e}'
    # a short call trains too (the chunk kernels take it), and eval mode builds no graph
    layer.zero_grad()
    short, _, _ = layer(xd[:, :8])
    short.sum().backward()
    assert layer.q_proj.weight.grad is not None
    assert not layer.eval()(xd)[0].requires_grad


def test_layer_missing_layer_idx():
    from fla_hip.layers import GatedDeltaNet, LayerCache
    layer = _layer()
    x = torch.randn(1, 8, 256, device=DEV, dtype=BF)
    layer.layer_idx = None
    with pytest.raises(ValueError):
        layer(x, past_key_values=LayerCache())
    with pytest.raises(ValueError):
        GatedDeltaNet(hidden_size=64, head_dim=16, num_heads=2, num_v_heads=3)


def test_decode_step_replayed_from_a_captured_graph():
    """A decode step of the layer captured once and replayed per token: the conv caches and the recurrent state are
    updated in place, so every replay continues from the previous one.  Checked against the same steps run eagerly."""
    from fla_hip.layers import LayerCache
    layer = _layer(seed=6)
    T, n = 100, 5
    x = torch.randn(2, T + n, 256, generator=torch.Generator().manual_seed(8)).to(BF).to(DEV)
    eager_cache = LayerCache()
    layer(x[:, :T], past_key_values=eager_cache, use_cache=True)
    eager = [layer(x[:, T + i:T + i + 1], past_key_values=eager_cache, use_cache=True)[0].clone() for i in range(n)]

    cache = LayerCache()
    layer(x[:, :T], past_key_values=cache, use_cache=True)
    state_ptr = cache[0]['recurrent_state'].data_ptr()
    token = x[:, T:T + 1].clone()                                # static input buffer of the graph
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                                # warm-up outside the capture, on a copy of the cache
        warm = LayerCache()
        warm.update(layer_idx=0, recurrent_state=cache[0]['recurrent_state'].clone(),
                    conv_state=tuple(c.clone() for c in cache[0]['conv_state']), offset=T)
        layer(token, past_key_values=warm, use_cache=True)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = layer(token, past_key_values=cache, use_cache=True)[0]
    # the capture itself does not run the step: the cache still holds the state after the prompt
    for i in range(n):
        token.copy_(x[:, T + i:T + i + 1])
        graph.replay()
        torch.cuda.synchronize()
        assert O.get_err_ratio(eager[i].float().cpu(), out.float().cpu()) < 1e-3, i
    assert cache[0]['recurrent_state'].data_ptr() == state_ptr
    assert torch.equal(cache[0]['recurrent_state'], eager_cache[0]['recurrent_state'])
