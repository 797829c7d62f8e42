"""CPU oracle for differential attention -- TEST INFRASTRUCTURE ONLY.

This file restates, in plain fp32/fp64 PyTorch, the materialised-softmax differential
attention of the reference (`src/layers.py:49-80`, function `MultiheadDiffAttn`).  It is the
checker that the HIP kernels are compared against.  Only the test-suite, the smoke check and the
benchmark's `cpu_baseline` leg may import it; the product path never does and has no CPU
fallback.

Deviations from the reference text, all deliberate:
  * everything is computed in `dtype` (fp32 by default, fp64 for gradcheck): the two `.half()`
    casts of `src/layers.py:65,68` are dropped, so the oracle is *stricter* than the reference;
  * apex `FusedRMSNorm(2*head_dim, elementwise_affine=False)` (`src/layers.py:75`; apex 0.1 is
    pinned in `requirements.txt:1` and is not vendored) is replaced by its published formula
    x * rsqrt(mean(x^2, -1) + eps) with apex's default eps = 1e-5, the same constant the
    reference kernel hard-codes (`src/kernel.py:50,197-198`);
  * the work is chunked over (batch, head) units, which are independent (`src/kernel.py:474`),
    to bound the N x N memory.

Pinned by (see tests/test_oracle.py): SDPA special cases, closed forms, a float64 brute-force
triple loop, float64 gradcheck, finite differences for d(lambda), and the identities between the
autograd backward and the explicit backward formulas below.
"""
import math

import torch

EPS = 1e-5  # apex FusedRMSNorm default; src/kernel.py:50


def _as_scalar(lambda_scale, dtype):
    if torch.is_tensor(lambda_scale):
        return lambda_scale.reshape(()).to(dtype)
    return torch.tensor(float(lambda_scale), dtype=dtype)


def _lambda_values(lambda_scale, H, dtype):
    """lambda as a vector: one value (the reference's case, src/layers.py:70) or one per head (not in
    the reference: each head then has its own lambda, shared over the batch)."""
    if torch.is_tensor(lambda_scale) and lambda_scale.numel() > 1:
        if lambda_scale.numel() != H:
            raise ValueError("lambda_scale must have 1 or H elements")
        return lambda_scale.reshape(H).to(dtype)
    return _as_scalar(lambda_scale, dtype).reshape(1)


def _lambda_of_units(lam_values, units, H):
    """[len(units), 1, 1] lambda of the (batch, head) units `units` (unit = b * H + h)."""
    if lam_values.numel() == 1:
        return lam_values.reshape(1, 1, 1)
    return lam_values[units % H].reshape(-1, 1, 1)


def normalise(x, lambda_init):
    """The rms_norm branch of src/layers.py:74-78 on pre-norm rows x [..., 2D]: apex's affine-free
    RMSNorm over the last dim (eps inside the root), then the (1 - lambda_init) factor.
    Returns (y, rinv) with rinv [..., 1]."""
    rinv = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + EPS)
    return (1 - lambda_init) * (x * rinv), rinv


def forward_unit(q1, q2, k1, k2, v, lam, lambda_init, rms_norm, want_aux=False, causal=False,
                 keep1=None, keep2=None, dropout_p=0.0):
    """One or more (b, h) units: tensors [..., N, D] / [..., N, 2D], already in the work dtype.

    Follows src/layers.py:60-78 line for line (minus the .half() casts).  `causal` (not in the
    reference, which lists masking as missing, src/kernel.py:4) lets query i see keys 0..i only, in
    both softmax streams.  Dropout (likewise listed as missing) takes its decisions as arguments,
    so the oracle stays deterministic: `keep1`, `keep2` [..., N, N] (non-zero = kept) multiply the
    two softmax maps after normalisation, and the kept entries are scaled by 1 / (1 - dropout_p),
    as torch's scaled_dot_product_attention defines dropout for its single map.
    """
    head_dim = q1.size(-1)
    sm_scale = 1 / math.sqrt(head_dim)                       # src/layers.py:60-62
    s1 = torch.matmul(q1, k1.transpose(-2, -1)) * sm_scale   # src/layers.py:64
    s2 = torch.matmul(q2, k2.transpose(-2, -1)) * sm_scale   # src/layers.py:67
    if causal:
        n = s1.size(-1)
        future = torch.ones(n, n, dtype=torch.bool, device=s1.device).triu(1)
        s1 = s1.masked_fill(future, float("-inf"))
        s2 = s2.masked_fill(future, float("-inf"))
    p1 = torch.softmax(s1, dim=-1)                           # src/layers.py:65
    p2 = torch.softmax(s2, dim=-1)                           # src/layers.py:68
    if keep1 is not None:
        p1 = p1 * keep1.to(p1.dtype) / (1 - dropout_p)
    if keep2 is not None:
        p2 = p2 * keep2.to(p2.dtype) / (1 - dropout_p)
    p = p1 - lam * p2                                        # src/layers.py:70
    x = torch.matmul(p, v)                                   # src/layers.py:72
    if rms_norm:                                             # src/layers.py:74-78
        y, rinv = normalise(x, lambda_init)
    else:
        rinv = None
        y = x
    if not want_aux:
        return y
    aux = {
        "x": x,
        "u1": torch.matmul(p1, v),
        "u2": torch.matmul(p2, v),
        "lse1": torch.logsumexp(s1, dim=-1),
        "lse2": torch.logsumexp(s2, dim=-1),
        "rinv": None if rinv is None else rinv.squeeze(-1),
    }
    return y, aux


def forward(q1, q2, k1, k2, v, lambda_scale, lambda_init=0.8, rms_norm=False,
            dtype=torch.float32, chunk=8, want_aux=False, causal=False, keep1=None, keep2=None, dropout_p=0.0):
    """Differential attention forward, [B,H,N,D] inputs, result in `dtype`.

    Inputs are upcast (fp16 values are used exactly as rounded).  `chunk` = number of (b,h)
    units processed together.  keep1, keep2: [B,H,N,N] dropout decisions (see forward_unit).
    """
    B, H, N, D = q1.shape
    Dv = v.shape[-1]
    f = lambda t: t.reshape(B * H, N, t.shape[-1]).to(dtype)
    q1f, q2f, k1f, k2f, vf = f(q1), f(q2), f(k1), f(k2), f(v)
    m1 = None if keep1 is None else keep1.reshape(B * H, N, N)
    m2 = None if keep2 is None else keep2.reshape(B * H, N, N)
    lam_values = _lambda_values(lambda_scale, H, dtype)
    ys, auxs = [], []
    for s in range(0, B * H, chunk):
        sl = slice(s, s + chunk)
        lam = _lambda_of_units(lam_values, torch.arange(s, min(s + chunk, B * H)), H)
        r = forward_unit(q1f[sl], q2f[sl], k1f[sl], k2f[sl], vf[sl], lam, lambda_init, rms_norm, want_aux, causal,
                         None if m1 is None else m1[sl], None if m2 is None else m2[sl], dropout_p)
        if want_aux:
            ys.append(r[0]); auxs.append(r[1])
        else:
            ys.append(r)
    y = torch.cat(ys).reshape(B, H, N, Dv)
    if not want_aux:
        return y
    aux = {}
    for key in auxs[0]:
        if auxs[0][key] is None:
            aux[key] = None
        else:
            t = torch.cat([a[key] for a in auxs])
            aux[key] = t.reshape(B, H, *t.shape[1:])
    return y, aux


def forward_backward(q1, q2, k1, k2, v, lambda_scale, dy, lambda_init=0.8, rms_norm=False,
                     dtype=torch.float32, chunk=8, causal=False, keep1=None, keep2=None, dropout_p=0.0):
    """Forward + autograd backward of the restated graph.

    Returns (y, dq1, dq2, dk1, dk2, dv, dlambda) in `dtype`; dlambda has shape [1] and is the sum
    over all (b,h) units (the reference sums its per-program partials the same way,
    src/kernel.py:573).  With one lambda per head, dlambda has shape [H]: the sum over the batch.
    """
    B, H, N, D = q1.shape
    Dv = v.shape[-1]
    f = lambda t: t.reshape(B * H, N, t.shape[-1]).to(dtype)
    ins = [f(q1), f(q2), f(k1), f(k2), f(v)]
    dyf = f(dy)
    lam0 = _lambda_values(lambda_scale, H, dtype)
    m1 = None if keep1 is None else keep1.reshape(B * H, N, N)
    m2 = None if keep2 is None else keep2.reshape(B * H, N, N)
    grads = [torch.empty_like(t) for t in ins]
    dlam = torch.zeros_like(lam0)
    ys = []
    for s in range(0, B * H, chunk):
        sl = slice(s, s + chunk)
        leaves = [t[sl].detach().clone().requires_grad_(True) for t in ins]
        lam_leaf = lam0.detach().clone().requires_grad_(True)
        lam = _lambda_of_units(lam_leaf, torch.arange(s, min(s + chunk, B * H)), H)
        y = forward_unit(*leaves, lam, lambda_init, rms_norm, causal=causal,
                         keep1=None if m1 is None else m1[sl], keep2=None if m2 is None else m2[sl], dropout_p=dropout_p)
        g = torch.autograd.grad(y, leaves + [lam_leaf], dyf[sl])
        for dst, src in zip(grads, g[:5]):
            dst[sl] = src
        dlam = dlam + g[5]
        ys.append(y.detach())
    y = torch.cat(ys).reshape(B, H, N, Dv)
    shp = lambda t: t.reshape(B, H, N, t.shape[-1])
    return (y, shp(grads[0]), shp(grads[1]), shp(grads[2]), shp(grads[3]), shp(grads[4]), dlam)


def backward_explicit(q1, q2, k1, k2, v, lambda_scale, dy, lambda_init=0.8, rms_norm=False,
                      dtype=torch.float32):
    """Backward by the closed formulas the fused kernels implement (no autograd), unchunked.

    Formulas: RMSNorm backward and row dots src/kernel.py:283-296; recompute of the probabilities
    from the row logsumexps :413-414; dV :416; dP :418; dS :420-421; dK :423-424; dQ :432-436.
    Differences from the reference text: d(lambda) is -sum(dX*U2) exactly (the reference divides
    the lambda-scaled product by (lambda + 1e-5), :293).
    """
    f = lambda t: t.to(dtype)
    q1, q2, k1, k2, v, g = f(q1), f(q2), f(k1), f(k2), f(v), f(dy)
    lam = _as_scalar(lambda_scale, dtype)
    D, Dv = q1.shape[-1], v.shape[-1]
    s = 1 / math.sqrt(D)
    s1 = torch.matmul(q1, k1.transpose(-2, -1)) * s
    s2 = torch.matmul(q2, k2.transpose(-2, -1)) * s
    lse1 = torch.logsumexp(s1, -1, keepdim=True)
    lse2 = torch.logsumexp(s2, -1, keepdim=True)
    a1 = torch.exp(s1 - lse1)
    a2 = torch.exp(s2 - lse2)
    u1 = torch.matmul(a1, v)
    u2 = torch.matmul(a2, v)
    x = u1 - lam * u2
    if rms_norm:
        c = 1 - lambda_init
        r = torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + EPS)
        dx = c * (r * g - (r ** 3 / Dv) * (g * x).sum(-1, keepdim=True) * x)
    else:
        dx = g
    dlam = -(dx * u2).sum().reshape(1)
    delta1 = (dx * u1).sum(-1, keepdim=True)
    delta2 = -lam * (dx * u2).sum(-1, keepdim=True)
    dp = torch.matmul(dx, v.transpose(-2, -1))
    ds1 = a1 * (dp - delta1)
    ds2 = a2 * (-lam * dp - delta2)
    dv = torch.matmul((a1 - lam * a2).transpose(-2, -1), dx)
    dq1 = s * torch.matmul(ds1, k1)
    dq2 = s * torch.matmul(ds2, k2)
    dk1 = s * torch.matmul(ds1.transpose(-2, -1), q1)
    dk2 = s * torch.matmul(ds2.transpose(-2, -1), q2)
    return dq1, dq2, dk1, dk2, dv, dlam
