"""Properties of the operator that hold at any size, checked on the GPU at the headline shape: they need no
oracle, so they cover every (batch, head) unit of the full problem at once."""
import pytest
import torch

from util import make_inputs

pytestmark = pytest.mark.gpu

B, H, N, D = 4, 32, 2048, 64


def run(tensors, dy, lam_value=0.5, rms=True):
    from layers import MultiheadDiffAttnKernel
    leaves = [t.detach().clone().requires_grad_(True) for t in tensors]
    lam = torch.tensor([lam_value], dtype=torch.float16, device="cuda", requires_grad=True)
    y = MultiheadDiffAttnKernel(*leaves, lambda_scale=lam, lambda_init=0.8, rms_norm=rms)
    y.backward(dy)
    torch.cuda.synchronize()
    return y.detach(), [t.grad for t in leaves], lam.grad


@pytest.fixture(scope="module")
def problem():
    print("property tests at B=%d H=%d N=%d D=%d" % (B, H, N, D), flush=True)
    return [t.cuda() for t in make_inputs(B, H, N, D, seed=2)]


def close(a, b, rel):
    scale = b.float().abs().max().item()
    return (a.float() - b.float()).abs().max().item() <= rel * scale


def test_permuting_the_keys_permutes_their_gradients_and_nothing_else(problem):
    q1, q2, k1, k2, v, dy = problem
    perm = torch.randperm(N, generator=torch.Generator().manual_seed(1)).cuda()
    y, g, dl = run((q1, q2, k1, k2, v), dy)
    yp, gp, dlp = run((q1, q2, k1[:, :, perm], k2[:, :, perm], v[:, :, perm]), dy)
    # only the order of summation over keys changes
    assert close(yp, y, 2e-3)
    assert close(gp[0], g[0], 5e-3) and close(gp[1], g[1], 5e-3)
    for i in (2, 3, 4):
        assert close(gp[i], g[i][:, :, perm], 5e-3), i
    assert abs(dlp.item() - dl.item()) <= 2e-2 * max(abs(dl.item()), 1.0)


def test_units_do_not_interact(problem):
    """Reversing the order of the (batch, head) units reverses the results: no unit's result depends on where
    it sits in the launch (the workgroup-to-unit maps of the kernels are not the identity)."""
    q1, q2, k1, k2, v, dy = problem
    flip = lambda t: t.flatten(0, 1).flip(0).reshape(t.shape).contiguous()
    y, g, dl = run((q1, q2, k1, k2, v), dy)
    yf, gf, dlf = run(tuple(flip(t) for t in (q1, q2, k1, k2, v)), flip(dy))
    assert torch.equal(yf, flip(y))
    for a, b in zip(gf, g):
        assert torch.equal(a, flip(b))
    assert abs(dlf.item() - dl.item()) <= 2e-2 * max(abs(dl.item()), 1.0)      # the partial sums are reordered


def test_without_the_norm_the_output_is_linear_in_v_and_the_gradients_in_dy(problem):
    q1, q2, k1, k2, v, dy = problem
    y, g, dl = run((q1, q2, k1, k2, v), dy, rms=False)
    y2, g2, dl2 = run((q1, q2, k1, k2, 2 * v), dy, rms=False)
    assert close(y2, 2 * y.float(), 2e-3)
    assert close(g2[4], g[4], 2e-3)                       # dv does not depend on v
    assert close(g2[0], 2 * g[0].float(), 5e-3)           # dq, dk scale with v through dP
    y3, g3, dl3 = run((q1, q2, k1, k2, v), 0.5 * dy, rms=False)
    assert torch.equal(y3, y)
    for a, b in zip(g3, g):
        assert close(a, 0.5 * b.float(), 2e-3)


def test_the_normalised_output_is_the_plain_one_divided_by_its_row_rms(problem):
    """The two forward variants against each other: y_norm = x * (1 - lambda_init) / sqrt(mean(x^2) + 1e-5),
    with x the output without the norm (rounded to 16 bits once more than inside the kernel)."""
    q1, q2, k1, k2, v, dy = problem
    x, _, _ = run((q1, q2, k1, k2, v), dy, rms=False)
    y, _, _ = run((q1, q2, k1, k2, v), dy, rms=True)
    x = x.float()
    want = x * torch.rsqrt(x.square().mean(-1, keepdim=True) + 1e-5) * (1 - 0.8)
    assert close(y, want, 5e-3)
    assert y.float().square().mean(-1).max().item() <= 0.04 * 1.01      # (1 - lambda_init)^2, less what epsilon takes
