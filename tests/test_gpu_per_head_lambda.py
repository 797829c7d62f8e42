"""One lambda per head (a tensor of H values instead of one; not in the reference): GPU parity against
the oracle, which is pinned for this case head by head against its single-lambda form."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu

CASES = [
    # B, H, N, D, rms, causal
    (2, 4, 256, 64, True, False),
    (3, 5, 384, 32, False, False),    # odd head count, N not a multiple of 256
    (1, 3, 256, 128, True, False),
    (2, 4, 200, 64, True, True),      # padded and causal
]


@pytest.mark.parametrize("B,H,N,D,rms,causal", CASES)
def test_per_head_lambda_matches_oracle(B, H, N, D, rms, causal):
    q1, q2, k1, k2, v, dy = make_inputs(B, H, N, D, seed=31)
    lams = [0.8 - 0.35 * h for h in range(H)]              # positive, zero-ish and negative values
    lam16 = torch.tensor(lams, dtype=torch.float16)
    print("case", B, H, N, D, rms, causal, flush=True)
    y, grads = run_kernel(q1, q2, k1, k2, v, lams, 0.8, rms, dy=dy, causal=causal)
    ref = orc.forward_backward(q1, q2, k1, k2, v, lam16, dy, 0.8, rms, causal=causal)
    assert max_abs(y, ref[0]) <= Y_ATOL
    for name, got, want in zip(("dq1", "dq2", "dk1", "dk2", "dv"), grads[:5], ref[1:6]):
        assert rel_to_max(got, want) <= GRAD_RTOL, name
    assert grads[5].shape == (H,)
    assert rel_to_max(grads[5], ref[6]) <= GRAD_RTOL


def test_equal_lambdas_give_the_single_lambda_result_bit_for_bit():
    B, H, N, D = 2, 4, 256, 64
    q1, q2, k1, k2, v, dy = make_inputs(B, H, N, D, seed=32)
    y1, g1 = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, dy=dy)
    yh, gh = run_kernel(q1, q2, k1, k2, v, [0.5] * H, 0.8, True, dy=dy)
    assert torch.equal(y1, yh)
    for a, b in zip(g1[:5], gh[:5]):
        assert torch.equal(a, b)
    # the single d(lambda) is the sum of the per-head ones, up to their fp16 rounding
    assert abs(g1[5].float().item() - gh[5].float().sum().item()) <= 4e-3 * max(1.0, abs(g1[5].float().item()))
