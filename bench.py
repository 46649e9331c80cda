"""Benchmark of the gated delta rule inference path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload prefill|prefill_b4|varlen|decode|decode_bf16_states|decode_v_first|decode_kda|ref_*|train_ref_*|chunk_kda|chunk_comba|train_chunk_kda|train_chunk_comba|layer_train|layer_steps|calib_copy|calib_rmw]

Prints ONE JSON line.  Default workload: chunked prefill, B=1, T=32768, Hqk=16, Hv=32,
K=V=128, bf16 inputs, fp32 state (random initial state, final state returned) - the
configuration the >= 50 %-of-MFMA-roofline target is quoted on.  A step is one call of
chunk_gated_delta_rule on inputs already resident in HBM.  The same line carries, under
"other_workloads" and in short form (ms per call, fraction of the bounding roofline), the reference's published
shapes (forward, and forward + backward through autograd: the `*_fwd_bwd` rows), the sibling operators, the layer's two
memory-bound steps either side of the operator (causal convolution, gated norm), the default workload again with exact
start states forced and with gates that hardly decay, and last the benchmark's other configurations (packed prefill, B=4
prefill, the decode step at B=256: us/step and state GB/s); and:
  roofline      dominant stage (the launches of one C entry point), algorithmic FLOPs (or bytes)
                per call / its mean duration measured with HIP events on the launch stream
  cpu_baseline  the CPU oracle (torch fp32, all host cores) on a bounded sample of the workload
Before the W warm-up steps of a workload the GPU is kept busy with the same step for 80 ms (untimed), so that the timed
steps run at the clocks of sustained load and not at those of the first milliseconds after an idle period;
"ms_per_step_cold" is the default workload timed without that (5 + 20 calls straight after an idle half second).
--workload layer_steps runs only the convolution and the gated norm; --workload calib_copy runs a plain 1 GiB device copy: the kernel of known size against which the
FETCH_SIZE / WRITE_SIZE counters of a profiler run are scaled; --workload calib_rmw an in-place read-modify-write of the decode states' 2 x 512 MiB
with torch's elementwise kernel: the stream the decode step is compared with.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, 'flash-linear-attention_amd')):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import torch  # noqa: E402
import torch.nn.functional as F  # noqa: E402

C, K, V = 64, 128, 128


def flops_per_unit(k, v):
    """Algorithmic FLOPs per (token, v-head) of the chunked gated delta rule as the reference evaluates it:
    2*(3CK + 2CV + 3KV) (K K^T, q k^T, w; u, P v_new; w S, k^T v_new, q S) = 180224 at K = V = 128.
    Here the sequential stage does k S, q S, k^T v_new (3KV), Xb D and P v_new (2CV); the rest (K K^T, q k^T, the
    64x64 inverse) is the chunk-parallel stage.  Returns (whole operator, sequential stage)."""
    return 2 * (3 * C * k + 2 * C * v + 3 * k * v), 2 * (3 * k * v + 2 * C * v)


def measured_traffic(key):
    """HBM bytes per launch of a workload's dominant stage as a profiler run of this file measured them (FETCH_SIZE +
    WRITE_SIZE scaled by the calib_copy workload): read from profiles/hbm_traffic.json, which names the run; None for
    workloads that have no such run.  Nothing is measured in the run that prints it."""
    try:
        with open(os.path.join(ROOT, 'profiles', 'hbm_traffic.json')) as fh:
            rec = json.load(fh)['workloads'].get(key)
        return None if rec is None else rec['dominant_stage_bytes']
    except (OSError, KeyError, ValueError):
        return None


PEAK_BF16_TFLOPS = 2500.0                      # MI355X dense bf16 MFMA, published
PEAK_HBM_GBS = 8000.0                          # MI355X HBM3E, published

WORKLOADS = {
    'prefill': dict(kind='prefill', B=1, T=32768, H=16, HV=32, h0=True, varlen=False,
                    name='configs[2]: GDN chunk prefill B=1 T=32768 Hqk=16 Hv=32 K=V=128 bf16, fp32 state'),
    'prefill_b4': dict(kind='prefill', B=4, T=4096, H=16, HV=16, h0=False, varlen=False,
                       name='configs[1]: GDN chunk prefill B=4 T=4096 H=16 K=V=128 bf16, fp32 state'),
    'varlen': dict(kind='prefill', B=1, T=65536, H=16, HV=32, h0=True, varlen=True,
                   name='configs[3]: GDN varlen prefill 65536 tokens in 32 sequences Hqk=16 Hv=32 K=V=128 bf16'),
    'decode': dict(kind='decode', N=256, H=16, HV=32,
                   name='configs[4]: GDN single-token decode batch=256 Hqk=16 Hv=32 K=V=128 bf16, fp32 states in place'),
    'decode_bf16_states': dict(kind='decode', N=256, H=16, HV=32, state_dtype='bf16',
                               name='the decode step of configs[4] with the states kept in bf16 (an option of this library: '
                                    'fp32 step, one rounding per step; 2 x 256 MiB of state traffic)'),
    'decode_v_first': dict(kind='decode', N=256, H=16, HV=32, v_first=True,
                           name='the decode step of configs[4] on V-first states [N,HV,V,K] (state_v_first, the layout serving engines keep)'),
    'decode_kda': dict(kind='decode', N=256, H=16, HV=32, op='kda',
                       name='the KDA operator\'s decode step (a decay per key feature) at the shape of configs[4]'),
    # configs[2] again, so that the headline's dependence on the gates is a number: with the exact start states of the
    # time segments forced (first pass, merge, second pass), and with gates that hardly decay (logsigmoid / 1024:
    # no segment can start from a zero state, so the automatic choice takes the exact path by itself)
    'prefill_exact': dict(kind='prefill', B=1, T=32768, H=16, HV=32, h0=True, varlen=False, scan_mode='segments-exact',
                          name='configs[2] with exact start states of the time segments (FLA_HIP_SCAN_MODE=segments-exact)'),
    'prefill_weak_decay': dict(kind='prefill', B=1, T=32768, H=16, HV=32, h0=True, varlen=False, gate_div=1024.0,
                               name='configs[2] with g = logsigmoid(N(0,1)) / 1024, automatic choice'),
}


def _published(B, T, H, D):
    return dict(kind='prefill', B=B, T=T, H=H, HV=H, K=D, V=D, h0=False, varlen=False, final=False, l2norm=True, raw_qk=True,
                name=f"the reference's published shape B={B} T={T} H={H} D={D} bf16: q, k not normalised, "
                     'use_qk_l2norm_in_kernel, no initial state, no final state')


# The shapes the reference publishes forward times for (benchmarks/ops/registry.py:323-335: H == HV, in-kernel l2 norm of
# raw q and k, no initial and no final state; README.md:566-580 adds D = 64 and D = 256): context rows, never `value`.
PUBLISHED = {
    'ref_b1_t8192_h96_d128': _published(1, 8192, 96, 128),
    'ref_b2_t16384_h16_d128': _published(2, 16384, 16, 128),
    'ref_b4_t2048_h16_d128': _published(4, 2048, 16, 128),
    'ref_b4_t4096_h64_d128': _published(4, 4096, 64, 128),
    'ref_b8_t1024_h8_d64': _published(8, 1024, 8, 64),
    'ref_b8_t2048_h32_d256': _published(8, 2048, 32, 256),
    # one long prompt through the reference layer's default head shape (fla/layers/gated_deltanet.py:91-92: head_dim 256, expand_v 2;
    # hidden size 2048 -> 6 heads): wide keys, time segments that start warm
    'layer_default_b1_t32768_h6_k256_v512': dict(kind='prefill', B=1, T=32768, H=6, HV=6, K=256, V=512, h0=False, varlen=False, final=True,
                                                 l2norm=True, raw_qk=True,
                                                 name="one prompt of 32768 tokens in the reference layer's default head shape: H=6 K=256 V=512 bf16, "
                                                      'use_qk_l2norm_in_kernel, final state returned'),
}
# ... and the same prompt with exact start states of the time segments forced: what a head pays whose gates decay too
# slowly for a warm start (first pass over 256-row states and transitions, merge, second pass)
PUBLISHED['layer_default_b1_t32768_h6_k256_v512_exact'] = dict(
    PUBLISHED['layer_default_b1_t32768_h6_k256_v512'], scan_mode='segments-exact',
    name=PUBLISHED['layer_default_b1_t32768_h6_k256_v512']['name'] + ', exact start states of the time segments')


def _ensure_built():
    from fla_hip import _lib
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()


def varlen_lengths(total, n_seq, lo, hi, seed=42):
    """configs[3]: lengths drawn uniformly in [lo, hi] from a seed, rescaled (floor) to sum to `total`, the remainder handed
    out one token at a time to the first sequences."""
    gen = torch.Generator().manual_seed(seed)
    L = torch.randint(lo, hi + 1, (n_seq,), generator=gen).double()
    L = torch.floor(L * total / L.sum()).long()
    for i in range(total - int(L.sum())):
        L[i % n_seq] += 1
    return [int(x) for x in L]


def make_prefill_inputs(w, device):
    gen = torch.Generator().manual_seed(42)
    B, T, H, HV = w['B'], w['T'], w['H'], w['HV']
    K, V = w.get('K', 128), w.get('V', 128)
    q, k = torch.randn(B, T, H, K, generator=gen), torch.randn(B, T, H, K, generator=gen)
    if not w.get('raw_qk'):
        q, k = F.normalize(q, p=2, dim=-1), F.normalize(k, p=2, dim=-1)
    q, k = q.bfloat16(), k.bfloat16()
    v = torch.randn(B, T, HV, V, generator=gen).bfloat16()
    g = F.logsigmoid(torch.randn(B, T, HV, generator=gen)) / w.get('gate_div', 16.0)
    beta = torch.sigmoid(torch.randn(B, T, HV, generator=gen))
    cu = None
    N = B
    if w['varlen']:
        lens = varlen_lengths(T, 32, 256, 4096, seed=42)
        cu = [0]
        for x in lens:
            cu.append(cu[-1] + x)
        N = 32
    h0 = 0.1 * torch.randn(N, HV, K, V, generator=gen) if w['h0'] else None
    cpu = dict(q=q, k=k, v=v, g=g, beta=beta, h0=h0, cu=cu)
    dev = {key: (val.to(device) if isinstance(val, torch.Tensor) else val) for key, val in cpu.items()}
    dev['cu_t'] = None if cu is None else torch.tensor(cu, dtype=torch.int64, device=device)
    dev['cu_cpu'] = None if cu is None else torch.tensor(cu, dtype=torch.int64)
    return cpu, dev


SPIN_UP_MS = 80.0


def spin_up(fn):
    """Untimed: repeat `fn` until the GPU has been busy for SPIN_UP_MS.  After an idle period (input generation, the CPU
    baseline of the previous workload) the first ~30 ms of sustained load run at lower clocks - measured here as 0.61 ms
    per call falling to 0.48 ms over the first 60 calls of the default workload - and a handful of warm-up steps
    does not cover that.  The W warm-up steps and the K timed steps follow as usual."""
    torch.cuda.synchronize()
    if SPIN_UP_MS <= 0:
        return
    t0 = time.perf_counter()
    i = 0
    while (time.perf_counter() - t0) * 1e3 < SPIN_UP_MS:
        fn(i) if fn.__code__.co_argcount else fn()
        i += 1
        if i % 8 == 0:
            torch.cuda.synchronize()
    torch.cuda.synchronize()


def bench_prefill(w, steps, warmup, device, with_cpu, cold=False):
    """One prefill workload.  `cold`: also time 20 calls (after 5) straight after the idle period of the input generation,
    before the untimed load that brings the clocks to those of sustained work ('ms_per_step_cold')."""
    mode = w.get('scan_mode')
    saved = os.environ.get('FLA_HIP_SCAN_MODE')
    if mode:
        os.environ['FLA_HIP_SCAN_MODE'] = mode       # (read by the operator when it builds its launch)
    try:
        return _bench_prefill(w, steps, warmup, device, with_cpu, cold)
    finally:
        if mode:
            if saved is None:
                os.environ.pop('FLA_HIP_SCAN_MODE', None)
            else:
                os.environ['FLA_HIP_SCAN_MODE'] = saved


def _bench_prefill(w, steps, warmup, device, with_cpu, cold):
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    from fla_hip.ops.gated_delta_rule.chunk import ChunkLaunch
    cpu, d = make_prefill_inputs(w, device)
    tokens = w['B'] * w['T']
    K, V = w.get('K', 128), w.get('V', 128)
    final, l2norm = w.get('final', True), w.get('l2norm', False)
    F_TOTAL, F_SCAN = flops_per_unit(K, V)
    F_PREP = F_TOTAL - F_SCAN

    def step():
        return chunk_gated_delta_rule(d['q'], d['k'], d['v'], d['g'], d['beta'], initial_state=d['h0'],
                                      output_final_state=final, use_qk_l2norm_in_kernel=l2norm,
                                      cu_seqlens=d['cu_t'], cu_seqlens_cpu=d['cu_cpu'])

    ms_cold = None
    if cold:
        torch.cuda.synchronize()
        time.sleep(0.5)
        for _ in range(5):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(20):
            step()
        torch.cuda.synchronize()
        ms_cold = (time.perf_counter() - t0) / 20 * 1e3
    spin_up(step)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / steps * 1e3

    # spread of single calls (HIP events around each; the reference's benchmarks report these quantiles,
    # benchmarks/ops/run.py:115-126)
    evq = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in evq:
        a.record()
        step()
        b.record()
    torch.cuda.synchronize()
    per_call = sorted(a.elapsed_time(b) for a, b in evq)
    quant = {f'p{int(100 * f)}': round(per_call[min(len(per_call) - 1, int(f * len(per_call)))], 4) for f in (0.2, 0.5, 0.8)}

    units = tokens * w['HV']
    whole = dict(flops=units * F_TOTAL, achieved=round(units * F_TOTAL / (elapsed / steps) / 1e12, 2),
                 frac=round(units * F_TOTAL / (elapsed / steps) / 1e12 / PEAK_BF16_TFLOPS, 5))
    if not w.get('stages', True):
        # context rows: the whole call against the matrix-core peak for the operator's algorithmic FLOPs
        roofline = dict(bound='mfma', achieved=whole['achieved'], peak=PEAK_BF16_TFLOPS, unit='TFLOP/s', frac=whole['frac'],
                        traffic=None, kernel='whole operator (all launches of one call)', kernel_us=round(ms_per_step * 1e3, 1),
                        flops_per_launch=whole['flops'])
        return dict(value=tokens * steps / elapsed, ms_per_step=ms_per_step, roofline=roofline, call_ms_quantiles=quant)
    # per-kernel durations: the same work issued as its two stages with HIP events in between
    call = ChunkLaunch(d['q'], d['k'], d['v'], d['g'], d['beta'], K ** -0.5, d['h0'], final, False,
                       d['cu_t'], d['cu_cpu'], None, 64, qk_l2norm=l2norm)
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for i in range(steps):
        ev[i][0].record()
        call.run('prepare')
        ev[i][1].record()
        call.run('scan')
        ev[i][2].record()
    torch.cuda.synchronize()
    t_prep = statistics.mean(e[0].elapsed_time(e[1]) for e in ev) * 1e-3
    t_scan = statistics.mean(e[1].elapsed_time(e[2]) for e in ev) * 1e-3
    scan_name = 'gdn_chunk_fwd_scan (all launches of the sequential stage)'
    dom = (scan_name, F_SCAN, t_scan) if t_scan >= t_prep else ('gdn_chunk_fwd_prepare: gdn_chunk_prepare_kernel', F_PREP, t_prep)
    achieved = units * dom[1] / dom[2] / 1e12
    roofline = dict(bound='mfma', achieved=round(achieved, 2), peak=PEAK_BF16_TFLOPS, unit='TFLOP/s',
                    frac=round(achieved / PEAK_BF16_TFLOPS, 5), traffic=measured_traffic(w['key']), kernel=dom[0],
                    kernel_us=round(dom[2] * 1e6, 1), flops_per_launch=units * dom[1],
                    kernels_us=dict(gdn_chunk_fwd_prepare=round(t_prep * 1e6, 1), gdn_chunk_fwd_scan=round(t_scan * 1e6, 1)),
                    whole_op=whole)
    out = dict(value=tokens * steps / elapsed, ms_per_step=ms_per_step, roofline=roofline, call_ms_quantiles=quant)
    if ms_cold is not None:
        out['ms_per_step_cold'] = round(ms_cold, 4)

    if with_cpu:
        out['cpu_baseline'] = cpu_baseline_prefill(w, cpu)
        # parity of this very workload's head of the sequence against the oracle
    return out


def bench_train(w, steps, warmup, device):
    """Forward and backward of the operator through autograd on one of the published shapes, as the reference times its
    'fwdbwd' mode (benchmarks/ops/run.py:340-384: the op, then backward of its output with a fixed do)."""
    from fla_hip.ops.gated_delta_rule import chunk_gated_delta_rule
    _, d = make_prefill_inputs(w, device)
    leaves = [d[n].requires_grad_(True) for n in ('q', 'k', 'v', 'g', 'beta')]
    do = torch.randn_like(d['v'])
    l2norm = w.get('l2norm', False)

    def step():
        o, _ = chunk_gated_delta_rule(*leaves, use_qk_l2norm_in_kernel=l2norm)
        o.backward(do)
        for x in leaves:
            x.grad = None

    per_call, _ = _time_calls(step, steps, warmup)
    return dict(workload=w['name'] + '; forward and backward through autograd', ms_per_step=round(per_call * 1e3, 4),
                tokens_per_s=round(w['B'] * w['T'] / per_call, 1))


def _train_step(op, leaves, do, **kw):
    def step():
        o, _ = op(*leaves, **kw)
        o.backward(do)
        for x in leaves:
            x.grad = None
    return step


def bench_kda(steps, warmup, device, train=False):
    """Chunked prefill of the sibling KDA operator (a decay per key feature) on one of the published GDN shapes; with
    ``train`` a training step (forward and backward through autograd)."""
    from fla_hip.ops.kda import chunk_kda
    B, T, H, D = 1, 8192, 96, 128
    gen = torch.Generator().manual_seed(42)
    q, k, v = (torch.randn(B, T, H, D, generator=gen).bfloat16().to(device) for _ in range(3))
    g = (F.logsigmoid(torch.randn(B, T, H, D, generator=gen)) / 4).to(device)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=gen)).to(device)
    call = lambda: chunk_kda(q, k, v, g, beta, use_qk_l2norm_in_kernel=True)
    if train:
        leaves = [x.requires_grad_(True) for x in (q, k, v, g, beta)]
        call = _train_step(chunk_kda, leaves, torch.randn_like(v), use_qk_l2norm_in_kernel=True)
    per_call, _ = _time_calls(call, steps, warmup)
    return dict(workload=f'chunk_kda {"forward and backward" if train else "forward"} B={B} T={T} H={H} K=V={D} bf16, fp32 log decays per key feature, in-kernel l2 norm',
                ms_per_step=round(per_call * 1e3, 4), tokens_per_s=round(B * T / per_call, 1))


def bench_comba(steps, warmup, device, train=False):
    """Chunked prefill of the sibling comba operator (a second key for the prediction) on one of the published GDN shapes; with
    ``train`` a training step (forward and backward through autograd)."""
    from fla_hip.ops.comba import chunk_comba
    B, T, H, D = 1, 8192, 96, 128
    gen = torch.Generator().manual_seed(42)
    q, k, v, p = (torch.randn(B, T, H, D, generator=gen).bfloat16().to(device) for _ in range(4))
    g = F.logsigmoid(torch.randn(B, T, H, generator=gen)).to(device)
    beta = torch.sigmoid(torch.randn(B, T, H, generator=gen)).to(device)
    call = lambda: chunk_comba(q, k, v, p, g, beta, use_qk_l2norm_in_kernel=True)
    if train:
        leaves = [x.requires_grad_(True) for x in (q, k, v, p, g, beta)]
        call = _train_step(chunk_comba, leaves, torch.randn_like(v), use_qk_l2norm_in_kernel=True)
    per_call, _ = _time_calls(call, steps, warmup)
    return dict(workload=f'chunk_comba {"forward and backward" if train else "forward"} B={B} T={T} H={H} K=V={D} bf16, fp32 log decays, in-kernel l2 norm of q, k, p',
                ms_per_step=round(per_call * 1e3, 4), tokens_per_s=round(B * T / per_call, 1))


def bench_layer_train(steps, warmup, device):
    """One training step (forward and backward) of the Gated DeltaNet layer with the reference's default sizes
    (fla/layers/gated_deltanet.py:88-107: hidden 2048, 6 heads of K = 256, V = 512, convolutions of size 4) on one prompt:
    torch matmuls for the projections, this library's kernels for everything between them, both ways."""
    from fla_hip.layers import GatedDeltaNet
    T = 32768
    torch.manual_seed(0)
    layer = GatedDeltaNet(hidden_size=2048, expand_v=2, head_dim=256, num_heads=6, layer_idx=0).to(device).bfloat16().train()
    x = torch.randn(1, T, 2048, device=device, dtype=torch.bfloat16, requires_grad=True)
    dy = torch.randn(1, T, 2048, device=device, dtype=torch.bfloat16)

    def step():
        out, _, _ = layer(x)
        out.backward(dy)
        x.grad = None
        layer.zero_grad(set_to_none=True)

    per_call, _ = _time_calls(step, steps, warmup)
    return dict(workload=f'GatedDeltaNet layer (hidden 2048, H=6, K=256, V=512, conv 4) forward + backward, one prompt of {T} tokens, bf16',
                ms_per_step=round(per_call * 1e3, 4), tokens_per_s=round(T / per_call, 1))


def cpu_baseline_prefill(w, cpu):
    """Oracle (torch fp32 chunked form) on the first tokens of the same inputs; the sample
    length is chosen from a short calibration run so that the timed run takes ~10-20 s."""
    from oracle import gdn_oracle as O
    torch.set_num_threads(os.cpu_count() or 1)

    def run(T_s):
        sl = slice(0, T_s)
        h0 = None if cpu['h0'] is None else cpu['h0'][:cpu['q'].shape[0]]
        t0 = time.perf_counter()
        O.chunk_gated_delta_rule(cpu['q'][:, sl], cpu['k'][:, sl], cpu['v'][:, sl], cpu['g'][:, sl], cpu['beta'][:, sl],
                                 None, h0, True)
        return time.perf_counter() - t0

    t_cal = run(512)
    rate = 512 * cpu['q'].shape[0] / t_cal
    T_s = int(min(cpu['q'].shape[1], max(1024, (rate * 12 / cpu['q'].shape[0]) // 64 * 64)))
    reps = max(1, min(8, int(12 / max(run(T_s), 1e-3))))          # about 10-20 s of CPU work in all
    ts = [run(T_s) for _ in range(reps)]
    t = statistics.median(ts)
    toks = T_s * cpu['q'].shape[0]
    return dict(value=round(toks / t, 1), unit='tokens/s', cores=torch.get_num_threads(), kind='port',
                sample=f'oracle chunk_gated_delta_rule (torch fp32 CPU), first {T_s} tokens of the same inputs, '
                       f'median of {reps} runs of {t:.1f} s', seconds=round(sum(ts), 2))


def bench_decode(w, steps, warmup, device, with_cpu):
    from fla_hip.ops.gated_delta_rule import fused_recurrent_gated_delta_rule
    N, H, HV = w['N'], w['H'], w['HV']
    gen = torch.Generator().manual_seed(42)
    q = F.normalize(torch.randn(N, 1, H, K, generator=gen), p=2, dim=-1).bfloat16()
    k = F.normalize(torch.randn(N, 1, H, K, generator=gen), p=2, dim=-1).bfloat16()
    v = torch.randn(N, 1, HV, V, generator=gen).bfloat16()
    kda = w.get('op') == 'kda'
    g = F.logsigmoid(torch.randn(N, 1, HV, K, generator=gen) if kda else torch.randn(N, 1, HV, generator=gen))
    beta = torch.sigmoid(torch.randn(N, 1, HV, generator=gen))
    h0 = 0.1 * torch.randn(N, HV, K, V, generator=gen)
    bf16_states = w.get('state_dtype') == 'bf16'
    if bf16_states:
        h0 = h0.bfloat16()
    dq, dk, dv, dg, db = (x.to(device) for x in (q, k, v, g, beta))
    # state pools used in turn: each step streams 2 x 512 MiB, more than the 256 MB Infinity Cache (bf16 states: four
    # pools of 256 MiB, so that a pool's lines have left the cache when its turn comes again)
    states = [h0.to(device) for _ in range(4 if bf16_states else 2)]

    v_first = bool(w.get('v_first'))
    if kda:
        from fla_hip.ops.kda import fused_recurrent_kda_fwd

    def step(i):
        if kda:
            return fused_recurrent_kda_fwd(dq, dk, dv, dg, db, initial_state=states[i % len(states)], output_final_state=True,
                                           inplace_final_state=True)
        return fused_recurrent_gated_delta_rule(dq, dk, dv, dg, beta=db, initial_state=states[i % len(states)],
                                                output_final_state=True, inplace_final_state=True, state_v_first=v_first)

    spin_up(step)
    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        step(i)
        ev[i + 1].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    t_kernel = statistics.mean(ev[i].elapsed_time(ev[i + 1]) for i in range(steps)) * 1e-3
    state_bytes = 2 * N * HV * K * V * h0.element_size()
    achieved = state_bytes / t_kernel / 1e9
    roofline = dict(bound='hbm', achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit='GB/s',
                    frac=round(achieved / PEAK_HBM_GBS, 4), traffic=measured_traffic(w['key']),
                    kernel='gdn_decode_bf16_kernel' if bf16_states else 'gdn_decode_vfirst_kernel' if v_first else 'gdn_decode_kernel',
                    kernel_us=round(t_kernel * 1e6, 1), bytes_per_launch=state_bytes)
    out = dict(value=elapsed / steps * 1e6, ms_per_step=elapsed / steps * 1e3, roofline=roofline)
    if with_cpu:
        from oracle import gdn_oracle as O
        torch.set_num_threads(os.cpu_count() or 1)
        S = h0.float()
        reps = 3
        t0 = time.perf_counter()
        for _ in range(reps):
            o_ref, S = O.decode_step(q[:, 0], k[:, 0], v[:, 0], g[:, 0], beta[:, 0], S)
        t = (time.perf_counter() - t0) / reps
        out['cpu_baseline'] = dict(value=round(t * 1e6, 1), unit='us/step', cores=torch.get_num_threads(), kind='port',
                                   sample=f'oracle decode_step (torch fp32 CPU), full batch of {N}, mean of {reps} steps',
                                   seconds=round(t * reps, 2))
    return out


def _time_calls(fn, steps, warmup):
    spin_up(fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    return elapsed / steps, statistics.mean(ev[i].elapsed_time(ev[i + 1]) for i in range(steps)) * 1e-3


def bench_layer_steps(steps, warmup, device, with_cpu):
    """The two memory-bound steps either side of the operator in the layer at the default prefill size: the causal
    convolution (+ SiLU) over the joined q|k|v projection (8192 channels, kernel size 4) and the gated RMS norm over
    the 32 value heads of 128 features.  Algorithmic bytes: every input element read once, every output written once."""
    from fla_hip.modules import causal_conv1d, causal_conv1d_bwd, layer_norm_gated_bwd, layer_norm_gated_fwd, rms_norm_gated
    T, H, HV, W = 32768, 16, 32, 4
    D = 2 * H * K + HV * V
    gen = torch.Generator(device=device).manual_seed(42)
    x = torch.randn(1, T, D, generator=gen, device=device).bfloat16()
    wt = torch.randn(D, W, generator=gen, device=device).bfloat16()
    o = torch.randn(T * HV, V, generator=gen, device=device).bfloat16()
    gate = torch.randn(T * HV, V, generator=gen, device=device).bfloat16()
    wn = torch.randn(V, generator=gen, device=device).bfloat16()
    dy_x, dy_o = torch.randn_like(x), torch.randn_like(o)
    _, _, rstd, _ = layer_norm_gated_fwd(o, gate, wn, None, 'swish', 1e-5, is_rms_norm=True)
    out = {}
    cases = (('conv_qkv', 'causal_conv1d_fwd_kernel', 2 * T * D * 2,
              f'causal conv + SiLU, T={T}, {D} channels (q|k|v), kernel size {W}, bf16',
              lambda: causal_conv1d(x, wt, activation='silu')),
             ('norm_gate', 'norm_gated_rows_kernel', 3 * T * HV * V * 2,
              f'gated RMS norm (swish), {T}x{HV} rows of {V} features, bf16',
              lambda: rms_norm_gated(o, gate, wn, None, 'swish', eps=1e-5)),
             # the backward passes (training): x, dy read and dx written; x, g, dy read and dx, dg written.  The time is the
             # whole call: the kernel and the sum over the rows of partial parameter gradients it leaves
             ('conv_qkv_bwd', 'causal_conv1d_bwd_kernel', 3 * T * D * 2,
              f'backward of the causal conv + SiLU, T={T}, {D} channels, kernel size {W}, bf16',
              lambda: causal_conv1d_bwd(x, dy_x, None, wt, activation='silu')),
             ('norm_gate_bwd', 'norm_gated_bwd_kernel', 5 * T * HV * V * 2,
              f'backward of the gated RMS norm (swish), {T}x{HV} rows of {V} features, bf16',
              lambda: layer_norm_gated_bwd(dy_o, o, gate, wn, None, 'swish', 1e-5, None, rstd, is_rms_norm=True)))
    for key, kernel, nbytes, name, fn in cases:
        wall, t_kernel = _time_calls(fn, steps, warmup)
        achieved = nbytes / t_kernel / 1e9
        out[key] = dict(workload=name, ms_per_step=round(wall * 1e3, 4), tokens_per_s=round(T / wall, 1),
                        roofline=dict(bound='hbm', achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit='GB/s',
                                      frac=round(achieved / PEAK_HBM_GBS, 4), traffic=measured_traffic(key), kernel=kernel,
                                      kernel_us=round(t_kernel * 1e6, 1), bytes_per_launch=nbytes))
    if with_cpu:
        from oracle import modules_oracle as MO
        torch.set_num_threads(os.cpu_count() or 1)
        Ts = 2048                                      # bounded sample: the first 2048 tokens
        xs, ws = x[:, :Ts].cpu(), wt.cpu()
        t0 = time.perf_counter()
        MO.causal_conv1d(xs, ws, activation='silu')
        t = time.perf_counter() - t0
        out['conv_qkv']['cpu_baseline'] = dict(value=round(Ts / t, 1), unit='tokens/s', cores=torch.get_num_threads(), kind='port',
                                               sample=f'oracle causal_conv1d (torch fp32 CPU) on the first {Ts} tokens', seconds=round(t, 2))
        os_, gs = o[:Ts * HV].cpu(), gate[:Ts * HV].cpu()
        t0 = time.perf_counter()
        MO.norm_gated(os_, gs, wn.cpu(), None, None, 1e-5, 'swish', True)
        t = time.perf_counter() - t0
        out['norm_gate']['cpu_baseline'] = dict(value=round(Ts / t, 1), unit='tokens/s', cores=torch.get_num_threads(), kind='port',
                                                sample=f'oracle norm_gated (torch fp32 CPU) on the first {Ts} tokens', seconds=round(t, 2))
    return out


def calib_copy(steps, warmup, device):
    """A plain device-to-device copy of 1 GiB (reads 1 GiB, writes 1 GiB per launch)."""
    n = 1 << 30
    src = torch.empty(n, dtype=torch.uint8, device=device).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(warmup):
        dst.copy_(src)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        dst.copy_(src)
    torch.cuda.synchronize()
    t = (time.perf_counter() - t0) / steps
    print(json.dumps(dict(metric='calib_copy_GBps', value=round(2 * n / t / 1e9, 1), unit='GB/s', bytes_read=n, bytes_written=n,
                          steps=steps, warmup=warmup)))


def calib_rmw(steps, warmup, device):
    """The decode step's traffic without its arithmetic: every fp32 element of two alternating 512 MiB pools (the size
    of the B = 256 decode states) read, changed and written back in place - by torch's elementwise kernel (the headline
    of this workload), and by the library's calibration kernel gdn_calib_rmw, which has the decode step's shape (64 KB
    per workgroup, a workgroup-wide reduction between the reads and the writes) with the placement of the workgroups as
    parameters.  What these reach is what a read-modify-write stream of that size reaches on the machine."""
    from fla_hip import _lib
    lib = _lib.load()
    n = 256 * 32 * 128 * 128
    pools = [torch.zeros(n, dtype=torch.float32, device=device) for _ in range(2)]
    stream = torch.cuda.current_stream().cuda_stream

    def timed(fn):
        spin_up(fn)
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        ev[0].record()
        for i in range(steps):
            fn(i)
            ev[i + 1].record()
        torch.cuda.synchronize()
        ts = sorted(ev[i].elapsed_time(ev[i + 1]) * 1e-3 for i in range(steps))
        return statistics.mean(ts), ts[len(ts) // 2]

    t, tm = timed(lambda i: pools[i & 1].add_(1.0))
    shapes = {}
    for run, per_cu in ((0, 0), (32, 0), (32, 1), (32, 2), (32, 3), (1024, 0), (1024, 2)):
        ts, _ = timed(lambda i: _lib.check(lib.gdn_calib_rmw(pools[i & 1].data_ptr(), n, run, per_cu, stream)))
        shapes[f'xcd_run={run},workgroups_per_cu={per_cu}'] = dict(us_per_pass=round(ts * 1e6, 1), GBps=round(2 * n * 4 / ts / 1e9, 1))
    print(json.dumps(dict(metric='calib_rmw_GBps', value=round(2 * n * 4 / t / 1e9, 1), unit='GB/s', us_per_pass=round(t * 1e6, 1),
                          us_median=round(tm * 1e6, 1), bytes_read=n * 4, bytes_written=n * 4, steps=steps, warmup=warmup,
                          frac_of_peak=round(2 * n * 4 / t / 1e9 / PEAK_HBM_GBS, 4), gdn_calib_rmw=shapes)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=100)
    ap.add_argument('--warmup', type=int, default=20)
    ap.add_argument('--workload', default='prefill', choices=list(WORKLOADS) + list(PUBLISHED) + ['train_' + n for n in PUBLISHED] + ['chunk_kda', 'chunk_comba', 'train_chunk_kda', 'train_chunk_comba', 'layer_train', 'layer_steps', 'calib_copy', 'calib_rmw'])
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-extra', action='store_true', help='skip the other workloads')
    ap.add_argument('--no-spin-up', action='store_true', help='no untimed load in front of the warm-up steps (clocks as after an idle period)')
    args = ap.parse_args()
    if args.no_spin_up:
        global SPIN_UP_MS
        SPIN_UP_MS = 0.0
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py: this build measures ONE GPU only (every sequence and v-head is independent, so more GPUs '
              'shard them with no communication); run it with --gpus 1.', file=sys.stderr)
        sys.exit(2)
    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    _ensure_built()
    device = 'cuda:0'
    torch.cuda.set_device(0)

    if args.workload == 'calib_copy':
        calib_copy(args.steps, args.warmup, device)
        return
    if args.workload == 'calib_rmw':
        calib_rmw(args.steps, args.warmup, device)
        return
    if args.workload == 'layer_steps':
        print(json.dumps(dict(metric='gdn_layer_steps', steps=args.steps, warmup=args.warmup, dtype='bf16', data='synthetic',
                              **bench_layer_steps(args.steps, args.warmup, device, not args.no_cpu_baseline))))
        return
    for key, val in WORKLOADS.items():
        val['key'] = key
    if args.workload in ('train_chunk_kda', 'train_chunk_comba'):
        r = (bench_kda if args.workload.endswith('kda') else bench_comba)(args.steps, args.warmup, device, train=True)
        print(json.dumps(dict(metric=args.workload[len('train_'):] + '_fwd_bwd_tokens_per_s', value=r['tokens_per_s'], unit='tokens/s',
                              higher_is_better=True, n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=r['ms_per_step'],
                              dtype='bf16', data='synthetic', config=dict(workload=r['workload'], chunk_size=64))))
        return
    if args.workload == 'chunk_kda':
        r = bench_kda(args.steps, args.warmup, device)
        print(json.dumps(dict(metric='kda_chunk_prefill_tokens_per_s', value=r['tokens_per_s'], unit='tokens/s', higher_is_better=True,
                              n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=r['ms_per_step'], dtype='bf16',
                              data='synthetic', config=dict(workload=r['workload'], chunk_size=64))))
        return
    if args.workload == 'layer_train':
        r = bench_layer_train(args.steps, args.warmup, device)
        print(json.dumps(dict(metric='gdn_layer_fwd_bwd_tokens_per_s', value=r['tokens_per_s'], unit='tokens/s', higher_is_better=True,
                              n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=r['ms_per_step'], dtype='bf16',
                              data='synthetic', config=dict(workload=r['workload'], chunk_size=64))))
        return
    if args.workload == 'chunk_comba':
        r = bench_comba(args.steps, args.warmup, device)
        print(json.dumps(dict(metric='comba_chunk_prefill_tokens_per_s', value=r['tokens_per_s'], unit='tokens/s', higher_is_better=True,
                              n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=r['ms_per_step'], dtype='bf16',
                              data='synthetic', config=dict(workload=r['workload'], chunk_size=64))))
        return
    if args.workload.startswith('train_'):
        name = args.workload[len('train_'):]
        r = bench_train(dict(PUBLISHED[name], key=name), args.steps, args.warmup, device)
        print(json.dumps(dict(metric='gdn_chunk_fwd_bwd_tokens_per_s', value=r['tokens_per_s'], unit='tokens/s', higher_is_better=True,
                              n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=r['ms_per_step'], dtype='bf16',
                              data='synthetic', config=dict(workload=r['workload'], chunk_size=64))))
        return
    if args.workload in PUBLISHED:
        w = dict(PUBLISHED[args.workload], key=args.workload, stages=False)
        r = bench_prefill(w, args.steps, args.warmup, device, False)
        print(json.dumps(dict(metric='gdn_chunk_prefill_tokens_per_s', value=round(r['value'], 1), unit='tokens/s', higher_is_better=True,
                              n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=round(r['ms_per_step'], 4), dtype='bf16',
                              data='synthetic', config=dict(workload=w['name'], chunk_size=64), roofline=r['roofline'],
                              call_ms_quantiles=r['call_ms_quantiles'])))
        return
    w = WORKLOADS[args.workload]
    if w['kind'] == 'prefill':
        res = bench_prefill(w, args.steps, args.warmup, device, not args.no_cpu_baseline, cold=True)
        line = dict(metric='gdn_chunk_prefill_tokens_per_s', value=round(res['value'], 1), unit='tokens/s', higher_is_better=True)
    else:
        res = bench_decode(w, args.steps, args.warmup, device, not args.no_cpu_baseline)
        line = dict(metric='gdn_decode_us_per_step', value=round(res['value'], 2), unit='us/step', higher_is_better=False)
    line.update(n_gpus=1, steps=args.steps, warmup=args.warmup, ms_per_step=round(res['ms_per_step'], 4), scaling='weak',
                vs_baseline=None, dtype='bf16', data='synthetic', config=dict(workload=w['name'], chunk_size=64),
                roofline=res['roofline'])
    for key in ('ms_per_step_cold', 'cpu_baseline', 'call_ms_quantiles'):
        if key in res:
            line[key] = res[key]
    if not args.no_extra:
        # The other rows are kept short (the whole line stays well under 8 KB) and the benchmark's other configurations come last.
        # Keys: ms = wall time per call, frac = fraction of the roofline that bounds the row (prefill rows: the whole
        # operator's algorithmic FLOPs against the bf16 matrix-core peak; streaming rows: algorithmic bytes against 8 TB/s),
        # frac_stage / us = the same for the dominant stage alone and the durations of the two stages (HIP events).
        extra = {}
        half, quarter = (max(10, args.steps // 2), max(3, args.warmup // 2)), (max(10, args.steps // 4), max(3, args.warmup // 4))
        for name, ww in PUBLISHED.items():
            r = bench_prefill(dict(ww, key=name, stages=False), *half, device, False)
            extra[name] = dict(ms=round(r['ms_per_step'], 4), frac=r['roofline']['frac'])
            torch.cuda.empty_cache()
        for name, ww in PUBLISHED.items():       # training step (forward + backward) on the same shapes
            extra[name + '_fwd_bwd'] = dict(ms=bench_train(dict(ww, key=name), *quarter, device)['ms_per_step'])
            torch.cuda.empty_cache()
        extra['chunk_kda_b1_t8192_h96_d128'] = dict(ms=bench_kda(*quarter, device)['ms_per_step'])
        extra['chunk_kda_b1_t8192_h96_d128_fwd_bwd'] = dict(ms=bench_kda(*quarter, device, train=True)['ms_per_step'])
        torch.cuda.empty_cache()
        extra['chunk_comba_b1_t8192_h96_d128'] = dict(ms=bench_comba(*quarter, device)['ms_per_step'])
        extra['chunk_comba_b1_t8192_h96_d128_fwd_bwd'] = dict(ms=bench_comba(*quarter, device, train=True)['ms_per_step'])
        torch.cuda.empty_cache()
        extra['layer_train_t32768'] = dict(ms=bench_layer_train(max(5, args.steps // 10), 3, device)['ms_per_step'])
        torch.cuda.empty_cache()
        for key, r in bench_layer_steps(args.steps, args.warmup, device, False).items():
            extra[key] = dict(ms=r['ms_per_step'], GBps=r['roofline']['achieved'], frac=r['roofline']['frac'])
        for name, ww in WORKLOADS.items():
            if name == args.workload:
                continue
            if ww['kind'] == 'prefill':
                r = bench_prefill(ww, args.steps, args.warmup, device, False)
                rf = r['roofline']
                e = dict(ms=round(r['ms_per_step'], 4), tokens_per_s=round(r['value'], 1), frac=rf['whole_op']['frac'],
                         frac_stage=rf['frac'], us=rf['kernels_us'], traffic=rf['traffic'])
            else:
                r = bench_decode(ww, args.steps, args.warmup, device, name == 'decode' and not args.no_cpu_baseline)
                rf = r['roofline']
                e = dict(us_per_step=round(r['value'], 2), state_GBps=rf['achieved'], frac=rf['frac'], kernel_us=rf['kernel_us'],
                         bytes_per_launch=rf['bytes_per_launch'], traffic=rf['traffic'])
                if 'cpu_baseline' in r:
                    e['cpu_baseline'] = {k2: r['cpu_baseline'][k2] for k2 in ('value', 'unit', 'cores', 'kind')}
            extra[name] = e
            torch.cuda.empty_cache()
        # the benchmark's packed prefill, B=4 prefill and decode configurations last
        for name in ('varlen', 'prefill_b4', 'decode'):
            if name in extra:
                extra[name] = extra.pop(name)
        line['other_workloads'] = extra
    print(json.dumps(line, separators=(',', ':')))


if __name__ == '__main__':
    main()
