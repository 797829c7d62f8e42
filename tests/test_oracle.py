"""Pins the CPU oracle (oracle/diff_attn_oracle.py) without importing the reference.

Each test is chosen so that a plausible restatement mistake (a dropped term, a wrong sign, a
transposed operand, eps in the wrong place, the (1 - lambda_init) factor applied without
rms_norm) fails at least one of them.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import brute_force
from oracle import diff_attn_oracle as orc


def rand_inputs(B, H, N, D, seed=0, dtype=torch.float64, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda d: (torch.randn(B, H, N, d, generator=g, dtype=torch.float32) * scale).to(dtype)
    return mk(D), mk(D), mk(D), mk(D), mk(2 * D)


def test_lambda_zero_is_sdpa():
    q1, q2, k1, k2, v = rand_inputs(2, 3, 40, 16, seed=1)
    y = orc.forward(q1, q2, k1, k2, v, 0.0, rms_norm=False, dtype=torch.float64)
    ref = F.scaled_dot_product_attention(q1, k1, v)
    assert torch.allclose(y, ref, atol=1e-12)
    y = orc.forward(q1, q2, k1, k2, v, 0.0, lambda_init=0.3, rms_norm=True, dtype=torch.float64)
    ref = 0.7 * F.rms_norm(ref, (32,), eps=1e-5)
    assert torch.allclose(y, ref, atol=1e-12)


def test_identical_streams():
    q1, _, k1, _, v = rand_inputs(1, 2, 33, 8, seed=2)
    ref = F.scaled_dot_product_attention(q1, k1, v)
    y = orc.forward(q1, q1, k1, k1, v, 0.25, rms_norm=False, dtype=torch.float64)
    assert torch.allclose(y, 0.75 * ref, atol=1e-12)
    y = orc.forward(q1, q1, k1, k1, v, 1.0, lambda_init=0.8, rms_norm=True, dtype=torch.float64)
    assert torch.count_nonzero(y) == 0


def test_zero_keys_gives_mean_of_v():
    q1, q2, k1, k2, v = rand_inputs(1, 2, 17, 8, seed=3)
    y = orc.forward(q1, q2, 0 * k1, 0 * k2, v, 0.4, rms_norm=False, dtype=torch.float64)
    ref = 0.6 * v.mean(dim=2, keepdim=True).expand_as(v)
    assert torch.allclose(y, ref, atol=1e-12)


def test_single_key():
    q1, q2, k1, k2, v = rand_inputs(2, 2, 1, 4, seed=4)
    y = orc.forward(q1, q2, k1, k2, v, -0.5, rms_norm=False, dtype=torch.float64)
    assert torch.allclose(y, 1.5 * v, atol=1e-12)


def test_rmsnorm_invariants():
    q1, q2, k1, k2, v = rand_inputs(1, 2, 24, 8, seed=5)
    lam, li = 0.5, 0.8
    x = orc.forward(q1, q2, k1, k2, v, lam, lambda_init=li, rms_norm=False, dtype=torch.float64)
    y = orc.forward(q1, q2, k1, k2, v, lam, lambda_init=li, rms_norm=True, dtype=torch.float64)
    m = x.pow(2).mean(-1)
    assert torch.allclose(y.pow(2).mean(-1), (1 - li) ** 2 * m / (m + 1e-5), rtol=1e-10)
    # without rms_norm there is no (1 - lambda_init) factor (src/layers.py:74-78)
    x2 = orc.forward(q1, q2, k1, k2, v, lam, lambda_init=0.1, rms_norm=False, dtype=torch.float64)
    assert torch.equal(x, x2)
    # scale invariance of the normalised output for mean-square >> eps
    y3 = orc.forward(q1, q2, k1, k2, 1000.0 * v, lam, lambda_init=li, rms_norm=True, dtype=torch.float64)
    y4 = orc.forward(q1, q2, k1, k2, 3000.0 * v, lam, lambda_init=li, rms_norm=True, dtype=torch.float64)
    assert torch.allclose(y3, y4, atol=1e-9)
    # eps sits inside the square root, added to the mean square
    tiny = orc.forward(q1, q2, k1, k2, 1e-6 * v, lam, lambda_init=li, rms_norm=True, dtype=torch.float64)
    assert torch.allclose(tiny, (1 - li) * (1e-6 * x) / math.sqrt(1e-5), rtol=1e-5, atol=0)


@pytest.mark.parametrize("rms", [False, True])
def test_brute_force_f64(rms):
    q1, q2, k1, k2, v = rand_inputs(1, 1, 7, 3, seed=6)
    y = orc.forward(q1, q2, k1, k2, v, 0.37, lambda_init=0.6, rms_norm=rms, dtype=torch.float64)
    ref = brute_force.forward_unit(*(t[0, 0].numpy() for t in (q1, q2, k1, k2, v)), 0.37, 0.6, rms)
    assert np.allclose(y[0, 0].numpy(), ref, atol=1e-12)


def test_aux_outputs():
    q1, q2, k1, k2, v = rand_inputs(1, 2, 19, 8, seed=7)
    y, aux = orc.forward(q1, q2, k1, k2, v, 0.3, rms_norm=True, dtype=torch.float64, want_aux=True)
    s = 1 / math.sqrt(8)
    assert torch.allclose(aux["lse1"], torch.logsumexp(s * q1 @ k1.transpose(-1, -2), -1), atol=1e-12)
    assert torch.allclose(aux["lse2"], torch.logsumexp(s * q2 @ k2.transpose(-1, -2), -1), atol=1e-12)
    assert torch.allclose(aux["u1"], F.scaled_dot_product_attention(q1, k1, v), atol=1e-12)
    assert torch.allclose(aux["u2"], F.scaled_dot_product_attention(q2, k2, v), atol=1e-12)
    assert torch.allclose(aux["x"], aux["u1"] - 0.3 * aux["u2"], atol=1e-12)
    assert torch.allclose(y, 0.2 * aux["x"] * aux["rinv"][..., None], atol=1e-12)


@pytest.mark.parametrize("rms", [False, True])
def test_gradcheck_f64(rms):
    q1, q2, k1, k2, v = rand_inputs(1, 1, 5, 2, seed=8)
    lam = torch.tensor(0.45, dtype=torch.float64)
    ins = [t[0].clone().requires_grad_(True) for t in (q1, q2, k1, k2, v)] + [lam.requires_grad_(True)]
    fn = lambda a, b, c, d, e, l: orc.forward_unit(a, b, c, d, e, l, 0.8, rms)
    assert torch.autograd.gradcheck(fn, ins, eps=1e-6, atol=1e-6)


@pytest.mark.parametrize("rms", [False, True])
def test_explicit_backward_matches_autograd(rms):
    q1, q2, k1, k2, v = rand_inputs(2, 2, 21, 8, seed=9)
    g = torch.Generator().manual_seed(10)
    dy = torch.randn(2, 2, 21, 16, generator=g, dtype=torch.float64)
    lam = torch.tensor([0.55], dtype=torch.float64)
    auto = orc.forward_backward(q1, q2, k1, k2, v, lam, dy, 0.8, rms, dtype=torch.float64, chunk=3)
    expl = orc.backward_explicit(q1, q2, k1, k2, v, lam, dy, 0.8, rms, dtype=torch.float64)
    for a, e in zip(auto[1:], expl):
        assert torch.allclose(a, e, atol=1e-11), (a - e).abs().max()


def test_lambda_zero_grads_match_sdpa():
    q1, q2, k1, k2, v = rand_inputs(1, 2, 16, 8, seed=11)
    g = torch.Generator().manual_seed(12)
    dy = torch.randn(1, 2, 16, 16, generator=g, dtype=torch.float64)
    out = orc.forward_backward(q1, q2, k1, k2, v, 0.0, dy, rms_norm=False, dtype=torch.float64)
    a, b, c = (t.clone().requires_grad_(True) for t in (q1, k1, v))
    ref = torch.autograd.grad(F.scaled_dot_product_attention(a, b, c), (a, b, c), dy)
    assert torch.allclose(out[1], ref[0], atol=1e-12)
    assert torch.allclose(out[3], ref[1], atol=1e-12)
    assert torch.allclose(out[5], ref[2], atol=1e-12)
    assert torch.count_nonzero(out[2]) == 0 and torch.count_nonzero(out[4]) == 0
    # d(lambda) = -sum(dX * U2) is still non-zero at lambda = 0
    u2 = F.scaled_dot_product_attention(q2, k2, v)
    assert torch.allclose(out[6], -(dy * u2).sum().reshape(1), atol=1e-11)


@pytest.mark.parametrize("rms", [False, True])
def test_dlambda_finite_difference(rms):
    q1, q2, k1, k2, v = rand_inputs(1, 2, 12, 4, seed=13)
    g = torch.Generator().manual_seed(14)
    dy = torch.randn(1, 2, 12, 8, generator=g, dtype=torch.float64)
    lam, h = 0.5, 1e-6
    out = orc.forward_backward(q1, q2, k1, k2, v, lam, dy, 0.8, rms, dtype=torch.float64)
    yp = orc.forward(q1, q2, k1, k2, v, lam + h, 0.8, rms, dtype=torch.float64)
    ym = orc.forward(q1, q2, k1, k2, v, lam - h, 0.8, rms, dtype=torch.float64)
    fd = ((yp - ym) * dy).sum() / (2 * h)
    assert abs(out[6].item() - fd.item()) < 1e-6 * max(1.0, abs(fd.item()))


def test_chunking_and_dtype():
    q1, q2, k1, k2, v = rand_inputs(2, 3, 16, 8, seed=15, dtype=torch.float16)
    a = orc.forward(q1, q2, k1, k2, v, 0.5, rms_norm=True, chunk=1)
    b = orc.forward(q1, q2, k1, k2, v, 0.5, rms_norm=True, chunk=6)
    assert a.dtype == torch.float32 and torch.allclose(a, b, atol=1e-6)
    lam = torch.tensor([0.5], dtype=torch.float16)
    c = orc.forward(q1, q2, k1, k2, v, lam, rms_norm=True)
    assert torch.allclose(a, c, atol=1e-6)


# ---- causal variant (not in the reference; pinned the same way) ---------------------------------
from util import make_inputs, max_abs  # noqa: E402

def test_causal_lambda_zero_is_causal_sdpa():
    q1, q2, k1, k2, v, _ = make_inputs(1, 2, 48, 16, 11)
    y = orc.forward(q1, q2, k1, k2, v, 0.0, 0.8, False, causal=True)
    ref = F.scaled_dot_product_attention(q1.float(), k1.float(), v.float(), is_causal=True)
    assert max_abs(y, ref) < 2e-5
    y = orc.forward(q1, q2, k1, k2, v, 0.0, 0.8, True, causal=True)
    assert max_abs(y, 0.2 * F.rms_norm(ref, (32,), eps=1e-5)) < 2e-5


def test_causal_prefix_property_and_first_row():
    # row i of the causal result depends on rows 0..i only: truncating the sequence changes nothing before the cut
    q1, q2, k1, k2, v, _ = make_inputs(1, 1, 40, 8, 12)
    lam = torch.tensor([0.6], dtype=torch.float16)
    full = orc.forward(q1, q2, k1, k2, v, lam, 0.8, False, causal=True)
    cut = orc.forward(*(t[:, :, :17] for t in (q1, q2, k1, k2, v)), lam, 0.8, False, causal=True)
    assert max_abs(full[:, :, :17], cut) < 1e-6
    # query 0 sees key 0 only: X_0 = (1 - lambda) v_0
    assert max_abs(full[:, :, 0], (1 - lam.float()) * v[:, :, 0].float()) < 1e-6


def test_causal_gradients_do_not_flow_from_the_past_to_future_keys():
    q1, q2, k1, k2, v, dy = make_inputs(1, 1, 24, 8, 13)
    dy = dy.clone(); dy[:, :, 10:] = 0          # only rows 0..9 receive gradient
    out = orc.forward_backward(q1, q2, k1, k2, v, 0.5, dy, 0.8, True, causal=True)
    for g in (out[3], out[4], out[5]):          # dk1, dk2, dv of keys 10.. are exactly zero
        assert g[:, :, 10:].abs().max().item() == 0.0
    assert out[3][:, :, :10].abs().max().item() > 0


def test_per_head_lambda_is_the_scalar_oracle_head_by_head():
    """One lambda per head (not in the reference): head h of the result, its gradients and d(lambda)[h]
    must be what the single-lambda oracle gives on that head alone, for every batch entry together."""
    B, H, N, D = 2, 3, 24, 8
    g = torch.Generator().manual_seed(11)
    mk = lambda d: torch.randn(B, H, N, d, generator=g, dtype=torch.float64)
    q1, q2, k1, k2, v, dy = mk(D), mk(D), mk(D), mk(D), mk(2 * D), mk(2 * D)
    lam = torch.tensor([0.3, -0.7, 1.2], dtype=torch.float64)
    for rms in (False, True):
        for causal in (False, True):
            full = orc.forward_backward(q1, q2, k1, k2, v, lam, dy, 0.8, rms, dtype=torch.float64, chunk=4, causal=causal)
            assert full[6].shape == (H,)
            y_fwd = orc.forward(q1, q2, k1, k2, v, lam, 0.8, rms, dtype=torch.float64, chunk=5, causal=causal)
            assert torch.allclose(y_fwd, full[0], rtol=0, atol=1e-12)
            for h in range(H):
                sl = (slice(None), slice(h, h + 1))
                one = orc.forward_backward(q1[sl], q2[sl], k1[sl], k2[sl], v[sl], lam[h], dy[sl], 0.8, rms,
                                           dtype=torch.float64, chunk=1, causal=causal)
                for a, b in zip(full[:6], one[:6]):
                    assert torch.allclose(a[sl], b, rtol=0, atol=1e-12)
                assert torch.allclose(full[6][h], one[6][0], rtol=1e-12, atol=1e-12)


# ---- dropout (explicit keep decisions) ---------------------------------------------------------------

def _keep_masks(B, H, N, p, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(B, H, N, N, generator=g) >= p), (torch.rand(B, H, N, N, generator=g) >= p)


def test_dropout_keeping_everything_only_rescales():
    q1, q2, k1, k2, v = rand_inputs(1, 2, 12, 4, seed=30)
    ones = torch.ones(1, 2, 12, 12, dtype=torch.bool)
    plain = orc.forward(q1, q2, k1, k2, v, 0.4, rms_norm=False, dtype=torch.float64)
    kept = orc.forward(q1, q2, k1, k2, v, 0.4, rms_norm=False, dtype=torch.float64, keep1=ones, keep2=ones, dropout_p=0.25)
    assert torch.allclose(kept, plain / 0.75, atol=1e-12)
    # with the norm the scale cancels (up to eps)
    a = orc.forward(q1, q2, k1, k2, v, 0.4, rms_norm=True, dtype=torch.float64)
    b = orc.forward(q1, q2, k1, k2, v, 0.4, rms_norm=True, dtype=torch.float64, keep1=ones, keep2=ones, dropout_p=0.25)
    assert torch.allclose(a, b, atol=1e-4)


def test_dropping_a_key_everywhere_is_zeroing_its_value_row():
    """Dropout acts after the softmax normalisation: dropping key j for every query, in both maps, removes
    v[j] from every output row without renormalising the other weights."""
    q1, q2, k1, k2, v = rand_inputs(2, 2, 10, 4, seed=31)
    keep = torch.ones(2, 2, 10, 10, dtype=torch.bool)
    keep[:, :, :, 3] = False
    keep[:, :, :, 7] = False
    got = orc.forward(q1, q2, k1, k2, v, 0.6, rms_norm=False, dtype=torch.float64, keep1=keep, keep2=keep, dropout_p=0.2)
    v0 = v.clone()
    v0[:, :, 3] = 0
    v0[:, :, 7] = 0
    want = orc.forward(q1, q2, k1, k2, v0, 0.6, rms_norm=False, dtype=torch.float64) / 0.8
    assert torch.allclose(got, want, atol=1e-12)


def test_dropout_masks_act_on_their_own_stream():
    """With lambda = 0 the second map's mask is irrelevant; with only the second map dropped entirely the
    result is the first map's attention alone."""
    q1, q2, k1, k2, v = rand_inputs(1, 2, 9, 4, seed=32)
    m1, m2 = _keep_masks(1, 2, 9, 0.3, seed=33)
    a = orc.forward(q1, q2, k1, k2, v, 0.0, dtype=torch.float64, keep1=m1, keep2=m2, dropout_p=0.3)
    b = orc.forward(q1, q2, k1, k2, v, 0.0, dtype=torch.float64, keep1=m1, keep2=~m2, dropout_p=0.3)
    assert torch.equal(a, b)
    none = torch.zeros_like(m2)
    c = orc.forward(q1, q2, k1, k2, v, 0.9, dtype=torch.float64, keep1=torch.ones_like(m1), keep2=none, dropout_p=0.0)
    assert torch.allclose(c, F.scaled_dot_product_attention(q1, k1, v), atol=1e-12)


@pytest.mark.parametrize("rms", [False, True])
def test_dropout_brute_force_f64(rms):
    q1, q2, k1, k2, v = rand_inputs(1, 1, 7, 3, seed=34)
    m1, m2 = _keep_masks(1, 1, 7, 0.4, seed=35)
    y = orc.forward(q1, q2, k1, k2, v, 0.37, lambda_init=0.6, rms_norm=rms, dtype=torch.float64, keep1=m1, keep2=m2, dropout_p=0.4)
    ref = brute_force.forward_unit(*(t[0, 0].numpy() for t in (q1, q2, k1, k2, v)), 0.37, 0.6, rms,
                                   keep=(m1[0, 0].numpy(), m2[0, 0].numpy()), dropout_p=0.4)
    assert np.allclose(y[0, 0].numpy(), ref, atol=1e-12)


def test_dropout_gradients_respect_the_masks():
    """A dropped (query, key) pair carries no gradient into v through that map: with lambda = 0, dv[j] only
    collects the queries that kept j; and gradcheck holds with the masks in place."""
    q1, q2, k1, k2, v = rand_inputs(1, 1, 6, 2, seed=36)
    m1, m2 = _keep_masks(1, 1, 6, 0.5, seed=37)
    m1[0, 0, :, 2] = False                     # nobody keeps key 2 in the first map
    dy = torch.randn(1, 1, 6, 4, dtype=torch.float64, generator=torch.Generator().manual_seed(38))
    out = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([0.0], dtype=torch.float64), dy, 0.8, False,
                               dtype=torch.float64, keep1=m1, keep2=m2, dropout_p=0.5)
    assert out[5][0, 0, 2].abs().max() == 0    # dv of key 2
    lam = torch.tensor(0.45, dtype=torch.float64, requires_grad=True)
    ins = [t[0].clone().requires_grad_(True) for t in (q1, q2, k1, k2, v)] + [lam]
    fn = lambda a, b, c, d, e, l: orc.forward_unit(a, b, c, d, e, l, 0.8, True, keep1=m1[0], keep2=m2[0], dropout_p=0.5)
    assert torch.autograd.gradcheck(fn, ins, eps=1e-6, atol=1e-6)
