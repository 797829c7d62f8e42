"""The operator under HIP graph capture: the C ABI neither allocates nor synchronises, so forward and
backward can be captured (here through torch.cuda.make_graphed_callables) and replayed.  Every replay is
compared bit for bit with the eager result, with eager work and a synchronisation between replays."""
import pytest
import torch

from util import make_inputs

pytestmark = pytest.mark.gpu


def test_graph_replays_match_eager():
    from layers import MultiheadDiffAttnKernel

    dev = torch.device("cuda:0")
    q1, q2, k1, k2, v, dy = (t.to(dev) for t in make_inputs(2, 4, 256, 64, seed=51))
    lam = torch.tensor([0.5], dtype=torch.float16, device=dev)

    def fn(a, b, c, d, e, l):
        return MultiheadDiffAttnKernel(a, b, c, d, e, lambda_scale=l, lambda_init=0.8, rms_norm=True)

    ins = tuple(t.clone().requires_grad_(True) for t in (q1, q2, k1, k2, v, lam))
    y0 = fn(*ins)
    y0.backward(dy)
    g0 = [t.grad.clone() for t in ins]
    sample = tuple(t.clone().requires_grad_(True) for t in (q1, q2, k1, k2, v, lam))
    graphed = torch.cuda.make_graphed_callables(fn, sample)
    for _ in range(3):
        for t in ins:
            t.grad = None
        y = graphed(*ins)
        y.backward(dy)
        torch.cuda.synchronize()
        assert torch.equal(y, y0)
        assert all(torch.equal(t.grad, g) for t, g in zip(ins, g0))
        _ = (q1 @ q1.transpose(-1, -2)).sum().item()      # eager work and a synchronisation between replays
