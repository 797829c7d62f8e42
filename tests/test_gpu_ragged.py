"""Sequence lengths that are not multiples of 128 (a restriction of the reference's kernels, src/kernel.py:4,
:527): the host pads, the forward ignores the padding keys, the backward is exact on the real rows.
Checked against the fp32 oracle at the unpadded length, with the tolerances of the other parity tests."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("N,D,rms,causal", [
    (1, 64, False, False),       # a single token: X = (1 - lambda) v
    (37, 64, True, False),
    (100, 32, False, False),
    (129, 64, True, False),      # one real row in the second block
    (200, 128, True, False),
    (333, 64, False, True),
    (450, 128, True, True),
    (1000, 64, True, False),
    (1000, 32, True, True),
])
def test_ragged_lengths_match_oracle(N, D, rms, causal):
    q1, q2, k1, k2, v, dy = make_inputs(1, 2, N, D, seed=31)
    y, grads = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, rms, dy, causal=causal)
    assert y.shape == v.shape and all(g.shape == t.shape for g, t in zip(grads[:5], (q1, q2, k1, k2, v)))
    ref = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([0.5], dtype=torch.float16), dy, 0.8, rms, chunk=1,
                               causal=causal)
    assert max_abs(y, ref[0]) <= Y_ATOL
    for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), grads, ref[1:]):
        if r.abs().max().item() < 1e-6:      # e.g. one token: the softmax of a single key has no gradient
            assert g.float().abs().max().item() <= 2e-3, name
        else:
            assert rel_to_max(g, r) <= GRAD_RTOL, name


@pytest.mark.parametrize("N", [1, 2, 3, 70])
@pytest.mark.parametrize("rms", [True, False])
def test_short_sequences_with_large_scores(N, rms):
    """With few real keys and scores of magnitude ~10 a row's logsumexp is often far below zero, so
    exp(0 - lse) of a padding key is huge: the backward must mask padding keys, not rely on their zero rows."""
    q1, q2, k1, k2, v, dy = make_inputs(4, 8, N, 32, seed=34, scale=3.0)
    y, grads = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, rms, dy)
    ref = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([0.5], dtype=torch.float16), dy, 0.8, rms, chunk=1)
    assert torch.isfinite(y).all() and max_abs(y, ref[0]) <= 3 * Y_ATOL      # |v| is three times the usual
    for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), grads, ref[1:]):
        assert torch.isfinite(g).all(), name
        # a single key has no softmax gradient and, with rms_norm, no d(lambda): what is left is the
        # rounding noise of operands three times the usual size
        tol = GRAD_RTOL * r.abs().max().item() if r.abs().max().item() >= 1e-3 else 2e-2
        assert max_abs(g, r) <= tol, name


def test_single_token_closed_form():
    q1, q2, k1, k2, v, _ = make_inputs(2, 3, 1, 64, seed=32)
    y, _ = run_kernel(q1, q2, k1, k2, v, 0.25, 0.8, False)
    assert max_abs(y, 0.75 * v.float()) <= 2e-3


def test_padding_does_not_leak_into_real_rows():
    # the result for 200 rows must not depend on what a caller stores behind them
    q1, q2, k1, k2, v, dy = make_inputs(1, 2, 256, 64, seed=33)
    cut = [t[:, :, :200].contiguous() for t in (q1, q2, k1, k2, v)]
    y_a, g_a = run_kernel(*cut, 0.5, 0.8, True, dy[:, :, :200].contiguous())
    views = [t[:, :, :200] for t in (q1, q2, k1, k2, v)]                  # non-contiguous views of longer tensors
    y_b, g_b = run_kernel(*views, 0.5, 0.8, True, dy[:, :, :200])
    assert torch.equal(y_a, y_b) and all(torch.equal(a, b) for a, b in zip(g_a, g_b))
