"""bfloat16 tensors (the reference hard-codes fp16, src/kernel.py:175-176) on the GPU against the fp32 oracle
evaluated on the same bf16-rounded inputs.  bf16 carries 8 significant bits against fp16's 11, so the
bounds are the fp16 ones scaled by 2^3 in the error unit: outputs within max-abs 6e-2 (values of order
1-4), gradients within 8e-2 of the max-norm of the oracle gradient."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu

BF16_Y_ATOL = 6e-2
BF16_GRAD_RTOL = 8e-2


@pytest.mark.parametrize("B,H,N,D,rms,causal", [
    (1, 2, 256, 64, True, False),
    (2, 2, 512, 64, False, False),
    (1, 2, 384, 32, True, True),
    (1, 2, 256, 128, True, False),
    (1, 1, 300, 64, True, False),      # padded length
])
def test_bf16_matches_oracle(B, H, N, D, rms, causal):
    ins = [t.bfloat16() for t in make_inputs(B, H, N, D, seed=61)]
    q1, q2, k1, k2, v, dy = ins
    y, grads = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, rms, dy, causal=causal)
    assert y.dtype == torch.bfloat16 and all(g.dtype == torch.bfloat16 for g in grads)
    ref = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([0.5]), dy, 0.8, rms, chunk=1, causal=causal)
    assert max_abs(y, ref[0]) <= BF16_Y_ATOL
    for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), grads, ref[1:]):
        assert rel_to_max(g, r) <= BF16_GRAD_RTOL, name


def test_mixed_dtypes_are_rejected():
    from layers import MultiheadDiffAttnKernel
    q1, q2, k1, k2, v, _ = [t.cuda() for t in make_inputs(1, 1, 128, 64, seed=62)]
    with pytest.raises(TypeError):
        MultiheadDiffAttnKernel(q1, q2, k1.bfloat16(), k2, v, lambda_scale=0.5)
    with pytest.raises(TypeError):
        MultiheadDiffAttnKernel(*(t.float() for t in (q1, q2, k1, k2, v)), lambda_scale=0.5)
