"""Writes tests/golden/gdn_scalar_cases.npz and tests/golden/gdn_scalar_cases_ext.npz.

The expected values come from a scalar, pure-python, float64 evaluation of the
gated delta rule written directly from its definition (one token at a time, one
multiply-add at a time):

    S[a][b] *= exp(g_t)
    r[b]     = sum_a S[a][b] * k_t[a]
    d[b]     = beta_t * (v_t[b] - r[b])
    S[a][b] += k_t[a] * d[b]
    o_t[b]   = scale * sum_a S[a][b] * q_t[a]

(the update order of fla/ops/gated_delta_rule/naive.py:50-59).  It shares no code
with oracle/gdn_oracle.py, so the fixtures catch slips in that restatement
(argument order, decay-before-delta, where `scale` is applied, GVA head
mapping, which tokens belong to which packed sequence).  Nothing from the
reference is imported or executed.  Run:  python tests/golden/make_golden.py

The second file holds cases for the optional arguments of the token recurrence
(fla/ops/gated_delta_rule/fused_recurrent.py:114-174): per-key decay gk, per-value decay gv,
a beta per value column, and for the pooled states of continuous batching /
speculative decoding (fla/ops/kda/fused_recurrent.py:131-145,203-219): start
from the slot of the last accepted token, leave the state after token t in the
slot named for (sequence, t).
"""
import math
import os

import numpy as np


def scalar_gdn(q, k, v, g, beta, scale, h0, cu):
    """q,k: [T][H][K]; v: [T][HV][V]; g,beta: [T][HV]; h0: [N][HV][K][V] or None;
    cu: packed sequence boundaries.  Returns o [T][HV][V], ht [N][HV][K][V]."""
    T, H, K = len(q), len(q[0]), len(q[0][0])
    HV, V = len(v[0]), len(v[0][0])
    grp = HV // H
    o = [[[0.0] * V for _ in range(HV)] for _ in range(T)]
    ht = []
    for n in range(len(cu) - 1):
        Sn = []
        for hv in range(HV):
            h = hv // grp
            S = [[(h0[n][hv][a][b] if h0 is not None else 0.0) for b in range(V)] for a in range(K)]
            for t in range(cu[n], cu[n + 1]):
                e = math.exp(g[t][hv])
                for a in range(K):
                    for b in range(V):
                        S[a][b] *= e
                d = [0.0] * V
                for b in range(V):
                    r = 0.0
                    for a in range(K):
                        r += S[a][b] * k[t][h][a]
                    d[b] = beta[t][hv] * (v[t][hv][b] - r)
                for a in range(K):
                    for b in range(V):
                        S[a][b] += k[t][h][a] * d[b]
                for b in range(V):
                    acc = 0.0
                    for a in range(K):
                        acc += S[a][b] * q[t][h][a]
                    o[t][hv][b] = scale * acc
            Sn.append(S)
        ht.append(Sn)
    return o, ht


def scalar_gdn_ext(q, k, v, g, gk, gv, beta, scale, cu, start_state, after_token=None):
    """As scalar_gdn with the optional decays gk [T][HV][K], gv [T][HV][V] (None: absent) and
    beta [T][HV][V] per value column.  start_state(n) -> [HV][K][V] initial state of sequence n;
    after_token(n, t_local, hv, S) is called with the state after every token."""
    T, H, K = len(q), len(q[0]), len(q[0][0])
    HV, V = len(v[0]), len(v[0][0])
    grp = HV // H
    o = [[[0.0] * V for _ in range(HV)] for _ in range(T)]
    ht = []
    for n in range(len(cu) - 1):
        S0 = start_state(n)
        Sn = []
        for hv in range(HV):
            h = hv // grp
            S = [[S0[hv][a][b] for b in range(V)] for a in range(K)]
            for t in range(cu[n], cu[n + 1]):
                for a in range(K):
                    for b in range(V):
                        e = g[t][hv] if g is not None else 0.0
                        if gk is not None:
                            e += gk[t][hv][a]
                        if gv is not None:
                            e += gv[t][hv][b]
                        S[a][b] *= math.exp(e)
                d = [0.0] * V
                for b in range(V):
                    r = 0.0
                    for a in range(K):
                        r += S[a][b] * k[t][h][a]
                    d[b] = beta[t][hv][b] * (v[t][hv][b] - r)
                for a in range(K):
                    for b in range(V):
                        S[a][b] += k[t][h][a] * d[b]
                for b in range(V):
                    acc = 0.0
                    for a in range(K):
                        acc += S[a][b] * q[t][h][a]
                    o[t][hv][b] = scale * acc
                if after_token is not None:
                    after_token(n, t - cu[n], hv, S)
            Sn.append(S)
        ht.append(Sn)
    return o, ht


CASES = {
    # name: (cu_seqlens, H, HV, K, V, with_h0, scale)
    'single_T5': ([0, 5], 1, 1, 2, 2, False, None),
    'gva_T70_h0': ([0, 70], 1, 2, 3, 2, True, 0.7),          # crosses a 64-token chunk boundary
    'varlen_h0': ([0, 3, 4, 9, 75], 2, 4, 2, 3, True, None),  # 1-token sequence, ragged tails
}


def main():
    rs = np.random.RandomState(20240607)
    out = {}
    for name, (cu, H, HV, K, V, with_h0, scale) in CASES.items():
        T, N = cu[-1], len(cu) - 1
        q = rs.randn(T, H, K)
        k = rs.randn(T, H, K)
        k /= np.sqrt((k * k).sum(-1, keepdims=True))
        v = rs.randn(T, HV, V)
        g = -np.log1p(np.exp(-rs.randn(T, HV)))           # logsigmoid
        beta = 1.0 / (1.0 + np.exp(-rs.randn(T, HV)))
        h0 = rs.randn(N, HV, K, V) if with_h0 else None
        sc = K ** -0.5 if scale is None else scale
        o, ht = scalar_gdn(q.tolist(), k.tolist(), v.tolist(), g.tolist(), beta.tolist(), sc,
                           h0.tolist() if with_h0 else None, cu)
        out[f'{name}.cu'] = np.array(cu, dtype=np.int64)
        out[f'{name}.scale'] = np.array(sc)
        for key, val in dict(q=q, k=k, v=v, g=g, beta=beta, o=np.array(o), ht=np.array(ht)).items():
            out[f'{name}.{key}'] = val
        if with_h0:
            out[f'{name}.h0'] = h0
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'gdn_scalar_cases.npz')
    np.savez_compressed(path, **out)
    print('wrote', path, os.path.getsize(path), 'bytes')


EXT_CASES = {
    # name: (cu_seqlens, H, HV, K, V, gk, gv, g)
    'gk_gv_vbeta': ([0, 6], 1, 2, 3, 2, True, True, True),
    'gk_only_varlen': ([0, 2, 7], 2, 2, 2, 3, True, False, False),
    'gv_vbeta_varlen': ([0, 4, 5, 9], 1, 3, 2, 2, False, True, True),
}


def main_ext():
    rs = np.random.RandomState(20250811)
    out = {}
    for name, (cu, H, HV, K, V, has_gk, has_gv, has_g) in EXT_CASES.items():
        T, N = cu[-1], len(cu) - 1
        q = rs.randn(T, H, K)
        k = rs.randn(T, H, K)
        k /= np.sqrt((k * k).sum(-1, keepdims=True))
        v = rs.randn(T, HV, V)
        g = -np.log1p(np.exp(-rs.randn(T, HV))) if has_g else None
        gk = -0.5 * rs.rand(T, HV, K) if has_gk else None
        gv = -0.5 * rs.rand(T, HV, V) if has_gv else None
        beta = 1.0 / (1.0 + np.exp(-rs.randn(T, HV, V)))          # a beta per value column
        h0 = rs.randn(N, HV, K, V)
        sc = K ** -0.5
        tl = lambda x: None if x is None else x.tolist()
        o, ht = scalar_gdn_ext(q.tolist(), k.tolist(), v.tolist(), tl(g), tl(gk), tl(gv), beta.tolist(), sc, cu,
                               lambda n: h0[n].tolist())
        out[f'{name}.cu'] = np.array(cu, dtype=np.int64)
        out[f'{name}.scale'] = np.array(sc)
        for key, val in dict(q=q, k=k, v=v, g=g, gk=gk, gv=gv, beta=beta, h0=h0, o=np.array(o), ht=np.array(ht)).items():
            if val is not None:
                out[f'{name}.{key}'] = val

    # pooled states, a slot per token: 3 sequences of 1..3 draft tokens, pool of 12 slots
    name = 'spec_pool'
    cu, H, HV, K, V, slots, TMAX = [0, 3, 4, 6], 1, 2, 2, 3, 12, 3
    T, N = cu[-1], len(cu) - 1
    q = rs.randn(T, H, K)
    k = rs.randn(T, H, K)
    k /= np.sqrt((k * k).sum(-1, keepdims=True))
    v = rs.randn(T, HV, V)
    g = -np.log1p(np.exp(-rs.randn(T, HV)))
    beta = 1.0 / (1.0 + np.exp(-rs.randn(T, HV)))
    pool = rs.randn(slots, HV, K, V)
    idx = rs.permutation(slots)[:N * TMAX].reshape(N, TMAX)      # distinct slots
    accepted = np.array([2, 1, 2])                                # start from slot [n][accepted-1]
    pool_after = pool.copy()

    def after(n, t, hv, S):
        pool_after[idx[n][t], hv] = np.array(S)

    beta_v = np.repeat(beta[:, :, None], V, axis=2)
    sc = 0.9
    o, _ = scalar_gdn_ext(q.tolist(), k.tolist(), v.tolist(), g.tolist(), None, None, beta_v.tolist(), sc, cu,
                          lambda n: pool[idx[n][accepted[n] - 1]].tolist(), after)
    out[f'{name}.cu'] = np.array(cu, dtype=np.int64)
    out[f'{name}.scale'] = np.array(sc)
    for key, val in dict(q=q, k=k, v=v, g=g, beta=beta, pool=pool, idx=idx.astype(np.int64), accepted=accepted.astype(np.int64),
                         o=np.array(o), pool_after=pool_after).items():
        out[f'{name}.{key}'] = val
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'gdn_scalar_cases_ext.npz')
    np.savez_compressed(path, **out)
    print('wrote', path, os.path.getsize(path), 'bytes')


if __name__ == '__main__':
    import sys
    if 'ext' not in sys.argv[1:]:
        main()
    if 'base' not in sys.argv[1:]:
        main_ext()
