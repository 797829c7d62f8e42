"""GPU parity at the full sizes of the benchmark configurations (2, 3 and 4).

The kernels run on the full problem.  (batch, head) units are independent, so the fp32 CPU oracle
is evaluated unit by unit: on every unit where it is affordable (configuration 2: all 128;
configuration 3: all 16), otherwise on 16 units that cover every batch entry and include middle
heads (configuration 4).  d(lambda) of the full-size run is compared with the oracle's sum over
exactly the units that enter it: all of them, or, through one lambda per head, the whole batch of
the heads that were evaluated.
"""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu

GRADS = ("dq1", "dq2", "dk1", "dk2", "dv")


def oracle_units(units, tensors, lam, lambda_init, rms, backward):
    """Oracle results for the listed (b, h) units, stacked as a [1, len(units), N, .] problem."""
    pick = lambda t: torch.stack([t[b, h] for b, h in units]).unsqueeze(0)
    sub = [pick(t) for t in tensors]
    lam16 = torch.tensor([lam], dtype=torch.float16)
    if backward:
        return pick, orc.forward_backward(*sub[:5], lam16, sub[5], lambda_init, rms, chunk=1)
    return pick, (orc.forward(*sub[:5], lam16, lambda_init, rms, chunk=1),)


def test_config2_headline_every_unit():
    B, H, N, D, lam, lambda_init = 4, 32, 2048, 64, 0.5, 0.8
    print("full-size case: configuration 2, all %d units against the oracle" % (B * H), flush=True)
    ins = make_inputs(B, H, N, D, seed=2)
    y, grads = run_kernel(*ins[:5], lam, lambda_init, True, ins[5])
    ref = orc.forward_backward(*ins[:5], torch.tensor([lam], dtype=torch.float16), ins[5], lambda_init, True, chunk=4)
    # unit by unit, so that a misplaced unit cannot hide behind the global maximum
    for b in range(B):
        for h in range(H):
            assert max_abs(y[b, h], ref[0][b, h]) <= Y_ATOL, ("y", b, h)
            for name, g, r in zip(GRADS, grads, ref[1:6]):
                assert rel_to_max(g[b, h], r[b, h]) <= GRAD_RTOL, (name, b, h)
    e = rel_to_max(grads[5], ref[6])
    print("  dlambda %.4f, oracle %.4f (all units), rel err %.3e" % (grads[5].item(), ref[6].item(), e), flush=True)
    assert e <= GRAD_RTOL


@pytest.fixture(scope="module")
def config3():
    """Configuration 3 inputs and the oracle's pre-norm rows for every unit (the expensive part, shared
    by the rms_norm on and off cases)."""
    B, H, N, D = 1, 16, 16384, 64
    ins = make_inputs(B, H, N, D, seed=3, scale=0.5, with_dy=False)
    print("full-size case: configuration 3, oracle forward of all %d units" % (B * H), flush=True)
    x = orc.forward(*ins[:5], torch.tensor([0.3], dtype=torch.float16), 0.8, False, chunk=1)
    return ins, x


@pytest.mark.parametrize("rms", [True, False])
def test_config3_long_sequence_forward_every_unit(config3, rms):
    ins, x = config3
    y, _ = run_kernel(*ins[:5], 0.3, 0.8, rms)
    ref = orc.normalise(x, 0.8)[0] if rms else x
    assert torch.isfinite(y).all()
    for h in range(x.shape[1]):
        e = max_abs(y[0, h], ref[0, h])
        assert e <= Y_ATOL, (h, e)
    print("  rms_norm=%s: y max-abs err %.3e" % (rms, max_abs(y, ref)), flush=True)


def test_config4_large_head_dim_sixteen_units():
    B, H, N, D, lam, lambda_init = 8, 32, 4096, 128, 0.8, 0.2
    print("full-size case: configuration 4, 16 units against the oracle", flush=True)
    ins = make_inputs(B, H, N, D, seed=4)
    y, grads = run_kernel(*ins[:5], lam, lambda_init, False, ins[5])
    assert torch.isfinite(y).all() and all(torch.isfinite(g).all() for g in grads)
    heads = (13, 30)                                     # every batch entry of two heads
    units = [(b, h) for h in heads for b in range(B)]
    pick, ref = oracle_units(units, ins, lam, lambda_init, False, True)
    for i, (b, h) in enumerate(units):
        assert max_abs(y[b, h], ref[0][0, i]) <= Y_ATOL, ("y", b, h)
        for name, g, r in zip(GRADS, grads, ref[1:6]):
            assert rel_to_max(g[b, h], r[0, i]) <= GRAD_RTOL, (name, b, h)
    # the same problem with one (equal) lambda per head: the tensors come out bit for bit the same,
    # and d(lambda) splits by head, so the two evaluated heads can be compared with the oracle's sums
    yh, gh = run_kernel(*ins[:5], [lam] * H, lambda_init, False, ins[5])
    assert torch.equal(yh, y) and all(torch.equal(a, b) for a, b in zip(gh[:5], grads[:5]))
    lam16 = torch.tensor([lam], dtype=torch.float16)
    for k, h in enumerate(heads):
        sub = [torch.stack([t[b, h] for b in range(B)]).unsqueeze(0) for t in ins]
        want = orc.forward_backward(*sub[:5], lam16, sub[5], lambda_init, False, chunk=1)[6].item()
        got = gh[5][h].item()
        print("  dlambda of head %d: %.4f, oracle %.4f" % (h, got, want), flush=True)
        assert abs(got - want) <= GRAD_RTOL * max(abs(want), 1.0)
    total = gh[5].float().sum().item()
    assert abs(total - grads[5].item()) <= 2e-2 * max(abs(total), 1.0)      # H fp16 roundings against one
