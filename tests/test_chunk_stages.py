"""The chunk-parallel stage on its own (gdn_chunk_fwd_prepare through the C ABI): its records are unpacked and
compared with what the mathematics fixes for each chunk - the gate cumsum, (I+L)^-1 by a library inverse in fp64,
and the gated q k^T - as the reference checks its own stage kernels one by one
(tests/ops/test_gdn_kernels.py:159-290, tests/ops/test_solve_tril.py:35-50, tests/ops/utils/test_cumsum.py:17-33).

Record layout (per chunk and value head, 11264 bytes): Xb at 0 and P at 5120 as 16x16x32 matrix-core operand
fragments - fragment (tt, sp) holds for lane l (c = l % 16, g = l // 16) row 16 tt + c and the columns
32 sp + 4 g + e (e < 4) and 32 sp + 16 + 4 g + e - 4 (e >= 4); the fragments that are identically zero are not
stored and two are stored as their first half; 256 fp32 of tables at 10240."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import gdn_oracle as O

pytestmark = pytest.mark.gpu

REC_BYTES, REC_X, REC_P, REC_TAB, REC_TAB2 = 12288, 0, 5120, 10240, 11264
FRAGS = [((0, 0), 0, True), ((1, 0), 512, False), ((2, 0), 1536, False), ((2, 1), 2560, True), ((3, 0), 3072, False), ((3, 1), 4096, False)]


def _unpack(rec: torch.Tensor, base: int, dtype) -> torch.Tensor:
    """64 x 64 matrix from the fragments at byte offset `base` of one record (uint8 tensor of REC_BYTES)."""
    out = torch.zeros(64, 64, dtype=torch.float64)
    lanes = torch.arange(64)
    c, g = lanes % 16, lanes // 16
    for (tt, sp), off, half in FRAGS:
        n = 4 if half else 8
        vals = rec[base + off: base + off + 64 * n * 2].view(dtype).view(64, n).double()
        for e in range(n):
            col = 32 * sp + 4 * g + e if e < 4 else 32 * sp + 16 + 4 * g + (e - 4)
            out[16 * tt + c, col] = vals[:, e]
    return out


def _records(call, num_chunks, HV):
    # the records are the last part of the workspace (behind the matrices of the time segments, if any)
    ws = call.workspace.cpu()
    return ws[ws.numel() - num_chunks * HV * REC_BYTES:].view(num_chunks, HV, REC_BYTES)


@pytest.mark.parametrize('B,T,H,HV,K,dtype,gate_div,l2', [
    (2, 128, 2, 2, 64, torch.bfloat16, 1.0, False),            # tests/ops/test_gdn_kernels.py:159-166
    (2, 128, 2, 4, 64, torch.bfloat16, 1.0, False),
    (1, 256, 4, 4, 32, torch.float16, 1.0, False),
    (2, 200, 2, 4, 128, torch.bfloat16, 16.0, True),           # ragged last chunk, row factors of the l2 norm
    (1, 63, 1, 1, 16, torch.float16, 4.0, False),              # tests/ops/test_solve_tril.py:22
    (2, 100, 2, 4, 64, torch.bfloat16, 4.0, True),            # head dims up to 64: the row factors 1/|q_t| are in the tables
    (1, 128, 1, 2, 32, torch.bfloat16, 2.0, 'long'),           # keys of length 1.7: beta |k|^2 > 2 stretches the state
])
def test_prepare_stage_against_closed_forms(B, T, H, HV, K, dtype, gate_div, l2, monkeypatch):
    from fla_hip.ops.gated_delta_rule.chunk import ChunkLaunch
    # the scan kernels form P themselves; the chunk-parallel stage leaves it in its records only on request
    monkeypatch.setenv('FLA_HIP_SCAN_MODE', 'record-p')
    has_P = True
    gen = torch.Generator().manual_seed(7)
    q = torch.randn(B, T, H, K, generator=gen)
    k = torch.randn(B, T, H, K, generator=gen)
    long_keys, l2 = l2 == 'long', l2 is True
    if not l2:
        q, k = F.normalize(q, dim=-1), F.normalize(k, dim=-1)
    if long_keys:
        k = 1.7 * k
    q, k = q.to(dtype), k.to(dtype)
    v = torch.randn(B, T, HV, K, generator=gen).to(dtype)
    g = F.logsigmoid(torch.randn(B, T, HV, generator=gen)) / gate_div
    beta = torch.sigmoid(torch.randn(B, T, HV, generator=gen))
    scale = K ** -0.5
    call = ChunkLaunch(q.cuda(), k.cuda(), v.cuda(), g.cuda(), beta.cuda(), scale, None, True, qk_l2norm=l2)
    call.run('prepare')
    torch.cuda.synchronize()
    NT = (T + 63) // 64
    recs = _records(call, B * NT, HV)
    # the transition bounds sit in front of the records (one float per chunk and value head, padded to 256 bytes)
    ws = call.workspace.cpu()
    nb = (B * NT * HV * 4 + 255) // 256 * 256
    bounds = ws[ws.numel() - B * NT * HV * REC_BYTES - nb:][:B * NT * HV * 4].view(torch.float32).view(B * NT, HV).double()
    qn, kn = (O.l2norm(q.double()), O.l2norm(k.double())) if l2 else (q.double(), k.double())
    G = HV // H
    for b in range(B):
        for it in range(NT):
            n = min(64, T - 64 * it)
            sl = slice(64 * it, 64 * it + n)
            for hv in range(HV):
                rec = recs[b * NT + it, hv]
                gc = torch.cumsum(g[b, sl, hv].double(), 0) / math.log(2)            # chunk-local, log2 units
                bt = beta[b, sl, hv].double()
                kk, qq = kn[b, sl, hv // G], qn[b, sl, hv // G]
                decay = torch.exp2(gc[:, None] - gc[None, :])
                L = torch.tril(bt[:, None] * (kk @ kk.T) * decay, -1)
                Xb_ref = torch.linalg.inv(torch.eye(n, dtype=torch.float64) + L) * bt[None, :]
                P_ref = scale * torch.tril((qq @ kk.T) * decay)
                Xb, P = _unpack(rec, REC_X, dtype), _unpack(rec, REC_P, dtype)
                assert O.get_err_ratio(Xb_ref, Xb[:n, :n]) < 3e-3, (b, it, hv)
                if has_P:
                    assert O.get_err_ratio(P_ref, P[:n, :n]) < 3e-3, (b, it, hv)
                    assert torch.equal(P, torch.tril(P))
                assert not Xb[:n, n:].any() and torch.equal(Xb, torch.tril(Xb))          # lower triangular, tail columns zero
                tab = rec[REC_TAB:REC_TAB + 1024].view(torch.float32).double()
                rk = 1.0 / torch.sqrt((k[b, sl, hv // G].double() ** 2).sum(-1) + 1e-6) if l2 else torch.ones(n, dtype=torch.float64)
                assert abs(tab[192].item() - gc[-1].item()) < 1e-4 * max(1.0, abs(gc[-1].item()))          # G_last
                assert torch.allclose(tab[128:128 + n], torch.exp2(gc) * rk, rtol=2e-5, atol=1e-30)          # 2^G (k rows)
                # scale 2^G (q rows); the row factors 1/|q_t| of the l2 norm are the scan's (it has q in LDS), not the records',
                # except for head dims up to 64 and wide keys on few (chunk, head) units
                rq = 1.0 / torch.sqrt((q[b, sl, hv // G].double() ** 2).sum(-1) + 1e-6) if (l2 and (K <= 64 or (K > 128 and B * NT * HV < 4096))) else torch.ones(n, dtype=torch.float64)
                assert torch.allclose(tab[64:64 + n], scale * torch.exp2(gc) * rq, rtol=2e-5, atol=1e-30)
                assert torch.allclose(tab[0:n], torch.exp2(gc[-1] - gc) * rk, rtol=2e-5, atol=1e-30)         # 2^(G_last - G)
                tab2 = rec[REC_TAB2:REC_TAB2 + 1024].view(torch.float32).double()                            # what P is formed from
                assert torch.allclose(tab2[0:n], gc, rtol=1e-5, atol=1e-5)
                assert torch.allclose(tab2[64:64 + n], scale * rq, rtol=2e-5) and torch.allclose(tab2[128:128 + n], rk, rtol=2e-5)
                # the bound: its closed form, and that it does bound the chunk's transition prod_t gamma_t (I - beta_t k_t k_t^T)
                k2 = (kk * kk).sum(-1)
                closed = gc[-1] + torch.log2(torch.clamp((1 - bt * k2).abs(), min=1.0)).sum()
                got = bounds[b * NT + it, hv].item()
                assert abs(got - closed.item()) < 1e-3 * max(1.0, abs(closed.item())), (got, closed.item())
                M = torch.eye(K, dtype=torch.float64)
                for t in range(n):
                    M = math.exp(g[b, 64 * it + t, hv].item()) * (M - bt[t] * torch.outer(kk[t], kk[t] @ M))
                assert math.log2(torch.linalg.matrix_norm(M, 2).item() + 1e-300) <= got + 1e-3


@pytest.mark.parametrize('B,T,H,HV', [(2, 300, 2, 4), (1, 4200, 1, 2)])
def test_the_two_stages_one_by_one_equal_the_whole_operator(B, T, H, HV):
    """gdn_chunk_fwd == gdn_chunk_fwd_prepare followed by gdn_chunk_fwd_scan on the same arguments (bit for bit)."""
    from fla_hip.ops.gated_delta_rule.chunk import ChunkLaunch
    q, k, v, g, beta, h0 = O.make_inputs(B, T, H, HV, 128, 128, seed=9, gate_div=8.0, h0_std=0.3, dtype=torch.bfloat16)
    args = [t.cuda() for t in (q, k, v, g, beta)]
    whole = ChunkLaunch(*args, 128 ** -0.5, h0.cuda(), True)
    whole.run()
    o1, ht1 = whole.results()
    split = ChunkLaunch(*args, 128 ** -0.5, h0.cuda(), True)
    split.run('prepare')
    split.run('scan')
    o2, ht2 = split.results()
    assert torch.equal(o1, o2) and torch.equal(ht1, ht2)
    ref_o, ref_ht = O.chunk_gated_delta_rule(q, k, v, g, beta, None, h0, True)
    assert O.get_err_ratio(ref_o, o2.float().cpu()) < 5e-3 and O.get_err_ratio(ref_ht, ht2.cpu()) < 5e-3
