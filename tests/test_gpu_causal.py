"""Causal masking (a feature the reference lists as missing, src/kernel.py:4) on the GPU against the fp32
oracle, same tolerances as the unmasked parity tests, plus the structural properties of the mask."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,H,N,D,rms,lam", [
    (1, 2, 128, 64, True, 0.5),      # a single key block: every sub-tile is on the diagonal
    (2, 2, 256, 64, True, 0.5),
    (1, 2, 384, 64, False, 0.3),     # N not a multiple of 256: four-wave dQ workgroups
    (1, 3, 1024, 64, True, 0.5),
    (1, 2, 512, 32, True, -0.4),
    (1, 2, 384, 128, True, 0.8),     # two-launch dK/dV
    (1, 1, 640, 128, False, 0.5),
])
def test_causal_matches_oracle(B, H, N, D, rms, lam):
    q1, q2, k1, k2, v, dy = make_inputs(B, H, N, D, seed=21)
    y, grads = run_kernel(q1, q2, k1, k2, v, lam, 0.8, rms, dy, causal=True)
    ref = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([lam], dtype=torch.float16), dy, 0.8, rms, chunk=1, causal=True)
    assert max_abs(y, ref[0]) <= Y_ATOL
    for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), grads, ref[1:]):
        assert rel_to_max(g, r) <= GRAD_RTOL, name


def test_causal_prefix_and_zero_gradient_structure():
    q1, q2, k1, k2, v, dy = make_inputs(1, 2, 512, 64, seed=22)
    y_full, _ = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, None, causal=True)
    cut = [t[:, :, :256].contiguous() for t in (q1, q2, k1, k2, v)]
    y_cut, _ = run_kernel(*cut, 0.5, 0.8, True, None, causal=True)
    # rows 0..255 see keys 0..255 only: the 512-token result restricted to them is the 256-token result
    assert max_abs(y_full[:, :, :256], y_cut) <= 2e-3
    dy2 = dy.clone(); dy2[:, :, 200:] = 0
    _, grads = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, dy2, causal=True)
    for g in grads[2:5]:                       # no gradient reaches keys after the last row that has one
        assert g[:, :, 200:].abs().max().item() == 0.0
    for g in grads[0:2]:                       # nor queries without upstream gradient
        assert g[:, :, 200:].abs().max().item() == 0.0


def test_unmasked_path_is_untouched_by_the_flag_default():
    q1, q2, k1, k2, v, dy = make_inputs(1, 2, 256, 64, seed=23)
    a = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, dy)
    b = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, dy, causal=False)
    assert torch.equal(a[0], b[0]) and all(torch.equal(x, y) for x, y in zip(a[1], b[1]))
    c = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, dy, causal=True)
    assert not torch.equal(a[0], c[0])
