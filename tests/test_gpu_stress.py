"""Numerical stress on the GPU: large logits (the lazily updated softmax reference must keep up), one-hot
attention rows, constant inputs, zero upstream gradient.  Same oracle, same tolerances."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu


def _check(q1, q2, k1, k2, v, dy, lam, rms, causal=False, y_atol=Y_ATOL):
    y, grads = run_kernel(q1, q2, k1, k2, v, lam, 0.8, rms, dy, causal=causal)
    ref = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([lam], dtype=torch.float16), dy, 0.8, rms, chunk=1,
                               causal=causal)
    assert torch.isfinite(y).all() and all(torch.isfinite(g).all() for g in grads)
    assert max_abs(y, ref[0]) <= y_atol
    for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), grads, ref[1:]):
        if r.abs().max().item() < 1e-6:
            assert g.float().abs().max().item() <= 2e-3, name
        else:
            assert rel_to_max(g, r) <= GRAD_RTOL, name


@pytest.mark.parametrize("scale,D", [(3.0, 64), (4.0, 32), (2.5, 128)])
def test_large_logits(scale, D):
    # scores of order scale^2 * sqrt(D): nearly one-hot softmax rows, row maxima that keep growing along the keys
    q1, q2, k1, k2, v, dy = make_inputs(1, 2, 512, D, seed=41)
    q1, q2, k1, k2 = (t * scale for t in (q1, q2, k1, k2))
    _check(q1.half(), q2.half(), k1.half(), k2.half(), v, dy, 0.5, True)


def test_growing_row_maximum():
    # keys sorted so that every later tile raises the row maximum: the rescale path runs on every tile
    q1, q2, k1, k2, v, dy = make_inputs(1, 1, 512, 64, seed=42)
    ramp = torch.linspace(0.2, 3.0, 512).reshape(1, 1, 512, 1)
    k1 = (k1.abs() * ramp).half(); q1 = q1.abs().half()
    _check(q1, q2, k1, k2, v, dy, 0.5, True)
    _check(q1, q2, k1, k2, v, dy, 0.5, False, causal=True)


def test_constant_inputs_and_zero_gradient():
    B, H, N, D = 1, 2, 256, 64
    one = torch.ones(B, H, N, D, dtype=torch.float16)
    v = torch.randn(B, H, N, 2 * D, generator=torch.Generator().manual_seed(43)).half()
    dy = torch.randn(B, H, N, 2 * D, generator=torch.Generator().manual_seed(44)).half()
    _check(one, one, one, one, v, dy, 0.5, False)            # uniform attention: X = (1 - lambda) mean(V)
    q1, q2, k1, k2, v, dy = make_inputs(B, H, N, D, seed=45)
    y, grads = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, torch.zeros_like(dy))
    assert all(g.abs().max().item() == 0 for g in grads)     # zero upstream gradient gives exactly zero gradients


@pytest.mark.parametrize("scale", [1024.0, 1e-3])
@pytest.mark.parametrize("D", [32, 64, 128])
def test_upstream_gradient_with_a_loss_scale(D, scale):
    """dy multiplied by 1024, as a gradient scaler does: dP - delta reaches 1e5, beyond the 16-bit range, while
    dS = P (dP - delta) and the gradients (about 2000) stay well inside it.  Gradients are linear in dy.
    And the other end: an upstream gradient of order 1e-3, whose dS values are fp16 subnormals."""
    q1, q2, k1, k2, v, dy = make_inputs(1, 2, 1024, D, seed=46)
    y, grads = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, (dy * scale).half())
    ref = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([0.5], dtype=torch.float16), dy, 0.8, True)
    for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv"), grads, ref[1:6]):
        assert torch.isfinite(g).all(), name
        assert rel_to_max(g.float() / scale, r) <= GRAD_RTOL, name


@pytest.mark.parametrize("D", [32, 64])
def test_lambda_gradient_under_a_loss_scale(D):
    """The lambda gradient sums over every row of every unit, so it leaves the fp16 range long before the
    other gradients do.  With lambda in fp32 the library reads it and returns its gradient in fp32: exact up
    to the usual tolerance whatever the loss scale.  With lambda in fp16 the gradient is rounded to fp16 as
    the reference's is (src/kernel.py:573) and saturates to infinity beyond 65504."""
    from layers import MultiheadDiffAttnKernel
    B, H, N, scale = 2, 4, 1024, 1024.0
    q1, q2, k1, k2, v, dy = make_inputs(B, H, N, D, seed=47)
    ref = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([0.5], dtype=torch.float16), dy, 0.8, True)
    want = ref[6].float().item() * scale
    assert abs(want) > 65504, "the case is meant to leave the fp16 range (got %g)" % want
    got = {}
    for dtype in (torch.float32, torch.float16):
        t = [x.cuda().requires_grad_(True) for x in (q1, q2, k1, k2, v)]
        lam = torch.tensor([0.5], dtype=dtype, device="cuda", requires_grad=True)
        y = MultiheadDiffAttnKernel(*t, lambda_scale=lam, lambda_init=0.8, rms_norm=True)
        y.backward((dy * scale).half().cuda())
        assert lam.grad.dtype == dtype and lam.grad.shape == lam.shape
        got[dtype] = lam.grad.float().item()
        for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv"), (x.grad for x in t), ref[1:6]):
            assert rel_to_max(g.float().cpu() / scale, r) <= GRAD_RTOL, name
    assert abs(got[torch.float32] - want) <= GRAD_RTOL * abs(want)
    assert got[torch.float16] == float("inf") * (1 if want > 0 else -1)      # the documented saturation


def test_single_key_rows_with_a_large_norm_factor_get_no_score_gradient():
    """Under the causal mask the first query sees one key: its softmax is 1 whatever q and k are, so dq of that
    row is exactly zero.  With lambda just above 1 the two streams nearly cancel there, the norm factor is
    large (rsqrt of a mean square near eps) and dX with it; dS = A (dP - delta) then cancels two large numbers,
    which only comes out when delta is formed from the same rounded dX that the products read."""
    from layers import MultiheadDiffAttnKernel

    B, H, N, D = 2, 1, 37, 64
    g = torch.Generator().manual_seed(5586)
    mk = lambda d, s=1.0: (torch.randn(B, H, N, d, generator=g) * s).half()
    q1, q2, k1, k2 = (mk(D, 2.0) for _ in range(4))
    v, dy = mk(2 * D), mk(2 * D)
    lam = torch.tensor([1.005], dtype=torch.float32)
    leaves = [t.cuda().requires_grad_(True) for t in (q1, q2, k1, k2, v)]
    lam_dev = lam.cuda().requires_grad_(True)
    y = MultiheadDiffAttnKernel(*leaves, lambda_scale=lam_dev, lambda_init=0.8, rms_norm=True, causal=True)
    y.backward(dy.cuda())
    torch.cuda.synchronize()
    ref = orc.forward_backward(q1, q2, k1, k2, v, lam, dy, 0.8, True, causal=True)
    assert max_abs(y.detach(), ref[0]) <= Y_ATOL
    for name, t, want in zip(("dq1", "dq2"), leaves[:2], ref[1:3]):
        assert want[:, :, 0].abs().max().item() == 0.0                     # the oracle agrees: no gradient
        first_row = t.grad[:, :, 0].float().abs().max().item()
        assert first_row <= 1e-2 * want.abs().max().item(), (name, first_row)
    for name, t, want in zip(("dk1", "dk2"), leaves[2:4], ref[3:5]):
        assert rel_to_max(t.grad, want) <= GRAD_RTOL, name
