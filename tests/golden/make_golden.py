"""Writes tests/golden/gdn_scalar_cases.npz.

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


if __name__ == '__main__':
    main()
