"""Float64 scalar-loop restatement of differential attention -- TEST INFRASTRUCTURE ONLY.

Independent of torch's matmul/softmax: plain Python loops over one (b, h) unit, used on tiny
shapes to pin `diff_attn_oracle.forward` (the materialised path of src/layers.py:49-80).
"""
import math

import numpy as np

EPS = 1e-5


def forward_unit(q1, q2, k1, k2, v, lam, lambda_init, rms_norm, keep=None, dropout_p=0.0):
    """q*, k*: [N, D] float64 arrays; v: [N, Dv].  Returns y [N, Dv].  `keep`: optional pair of [N, N]
    0/1 arrays, the dropout decisions of the two softmax maps (kept entries scaled by 1/(1-p))."""
    n, d = q1.shape
    dv = v.shape[1]
    scale = 1.0 / math.sqrt(d)
    y = np.zeros((n, dv), dtype=np.float64)
    for i in range(n):
        rows = []
        for t_, (q, k) in enumerate(((q1, k1), (q2, k2))):
            sc = [scale * sum(q[i, t] * k[j, t] for t in range(d)) for j in range(n)]
            mx = max(sc)
            ex = [math.exp(x - mx) for x in sc]
            z = sum(ex)
            row = [e / z for e in ex]
            if keep is not None:
                row = [a / (1.0 - dropout_p) if keep[t_][i, j] else 0.0 for j, a in enumerate(row)]
            rows.append(row)
        x = [sum((rows[0][j] - lam * rows[1][j]) * v[j, c] for j in range(n)) for c in range(dv)]
        if rms_norm:
            ms = sum(t * t for t in x) / dv
            r = 1.0 / math.sqrt(ms + EPS)
            x = [(1.0 - lambda_init) * t * r for t in x]
        y[i, :] = x
    return y
