"""GPU parity at the full sizes of the benchmark configurations (2, 3 and 4).

The CPU oracle cannot afford every (batch, head) unit at these sizes, and units are independent,
so: the kernels run on the full problem; two units are checked against the fp32 oracle; the same
two units are run again as a B=1,H=2 problem, which must reproduce the full run bit for bit
(same tiles, same order) and whose d(lambda) is compared with the oracle's.
"""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu


def check_full(B, H, N, D, seed, lam, lambda_init, rms, scale, backward):
    print("full-size case", dict(B=B, H=H, N=N, D=D, seed=seed, lam=lam, rms=rms, backward=backward), flush=True)
    q1, q2, k1, k2, v, dy = make_inputs(B, H, N, D, seed, scale)
    y, grads = run_kernel(q1, q2, k1, k2, v, lam, lambda_init, rms, dy if backward else None)
    assert torch.isfinite(y).all()
    units = [(0, 0), (B - 1, H - 1)]
    pick = lambda t: torch.stack([t[b, h] for b, h in units]).unsqueeze(0).contiguous()
    sub = [pick(t) for t in (q1, q2, k1, k2, v, dy)]
    lam16 = torch.tensor([lam], dtype=torch.float16)
    if backward:
        ref = orc.forward_backward(*sub[:5], lam16, sub[5], lambda_init, rms, chunk=1)
    else:
        ref = (orc.forward(*sub[:5], lam16, lambda_init, rms, chunk=1),)
    e = max_abs(pick(y), ref[0])
    print("  y max-abs err %.3e" % e, flush=True)
    assert e <= Y_ATOL
    ys, gs = run_kernel(*sub[:5], lam, lambda_init, rms, sub[5] if backward else None)
    assert torch.equal(ys, pick(y)), "a unit's output must not depend on the other units in the launch"
    if backward:
        for name, g, gsub, r in zip(("dq1", "dq2", "dk1", "dk2", "dv"), grads, gs, ref[1:6]):
            assert torch.isfinite(g).all(), name
            assert torch.equal(gsub, pick(g)), name
            e = rel_to_max(pick(g), r)
            print("  %s rel-to-max err %.3e" % (name, e), flush=True)
            assert e <= GRAD_RTOL, name
        e = rel_to_max(gs[5], ref[6])
        print("  dlambda (two-unit problem) rel err %.3e (ref %.3e)" % (e, ref[6].item()), flush=True)
        assert e <= GRAD_RTOL
        assert torch.isfinite(grads[5]).all()


def test_config2_headline():
    check_full(4, 32, 2048, 64, seed=2, lam=0.5, lambda_init=0.8, rms=True, scale=1.0, backward=True)


@pytest.mark.parametrize("rms", [True, False])
def test_config3_long_sequence_forward(rms):
    check_full(1, 16, 16384, 64, seed=3, lam=0.3, lambda_init=0.8, rms=rms, scale=0.5, backward=False)


def test_config4_large_head_dim():
    check_full(8, 32, 4096, 128, seed=4, lam=0.8, lambda_init=0.2, rms=False, scale=1.0, backward=True)
