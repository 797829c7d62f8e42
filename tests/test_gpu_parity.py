"""GPU parity: the HIP kernels, called through layers.MultiheadDiffAttnKernel -> C ABI, against
the fp32 CPU oracle on the same seeded inputs."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu

GRAD_NAMES = ("dq1", "dq2", "dk1", "dk2", "dv", "dlambda")


def check_case(B, H, N, D, seed, lam, lambda_init, rms, scale=1.0, backward=True):
    q1, q2, k1, k2, v, dy = make_inputs(B, H, N, D, seed, scale)
    print("case", dict(B=B, H=H, N=N, D=D, seed=seed, lam=lam, rms=rms, backward=backward), flush=True)
    y, grads = run_kernel(q1, q2, k1, k2, v, lam, lambda_init, rms, dy if backward else None)
    lam16 = torch.tensor([lam], dtype=torch.float16)
    if backward:
        ref = orc.forward_backward(q1, q2, k1, k2, v, lam16, dy, lambda_init, rms)
    else:
        ref = (orc.forward(q1, q2, k1, k2, v, lam16, lambda_init, rms),)
    err_y = max_abs(y, ref[0])
    print("  y max-abs err %.3e" % err_y, flush=True)
    assert torch.isfinite(y).all()
    assert err_y <= Y_ATOL
    if backward:
        for name, gk, gr in zip(GRAD_NAMES, grads, ref[1:]):
            e = rel_to_max(gk, gr)
            print("  %s rel-to-max err %.3e (ref max %.3e)" % (name, e, gr.abs().max().item()), flush=True)
            assert torch.isfinite(gk).all(), name
            assert e <= GRAD_RTOL, name


@pytest.mark.parametrize("D", [32, 64, 128])
@pytest.mark.parametrize("rms", [True, False])
def test_small_forward_backward(D, rms):
    check_case(1, 2, 256, D, seed=100 + D, lam=0.5, lambda_init=0.8, rms=rms)


@pytest.mark.parametrize("D,N", [(32, 128), (64, 384), (128, 128), (64, 640)])
def test_odd_tile_counts(D, N):
    check_case(2, 1, N, D, seed=7 * D + N, lam=0.3, lambda_init=0.5, rms=True)


def test_config0_forward():
    # benchmark configuration 0: B=2 H=16 N=512 D=32, lambda 0.5, lambda_init 0.8, rms_norm on, forward only
    check_case(2, 16, 512, 32, seed=0, lam=0.5, lambda_init=0.8, rms=True, backward=False)


def test_config1_forward_backward():
    # benchmark configuration 1: same shape and inputs as config 0, forward + backward
    check_case(2, 16, 512, 32, seed=0, lam=0.5, lambda_init=0.8, rms=True, backward=True)


def test_negative_and_zero_lambda():
    check_case(1, 2, 256, 64, seed=5, lam=-0.5, lambda_init=0.8, rms=True)
    check_case(1, 2, 256, 64, seed=6, lam=0.0, lambda_init=0.8, rms=False)


def test_lambda_init_close_to_one():
    """The backward rebuilds the pre-norm row as Y / ((1 - lambda_init) * rinv) from the 16-bit Y: with
    lambda_init = 0.99 the stored Y is a hundred times smaller than usual."""
    check_case(1, 2, 256, 64, seed=21, lam=0.5, lambda_init=0.99, rms=True)
    check_case(1, 2, 128, 32, seed=22, lam=0.3, lambda_init=0.99, rms=True)


def test_backward_is_deterministic():
    q1, q2, k1, k2, v, dy = make_inputs(2, 4, 512, 64, seed=11)
    a = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, dy)
    b = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, dy)
    assert torch.equal(a[0], b[0])
    for ga, gb in zip(a[1], b[1]):
        assert torch.equal(ga, gb)


def test_second_derivative_is_refused():
    """The backward is a set of kernels without a derivative of its own: asking autograd to differentiate
    through it must raise instead of returning zeros."""
    from layers import MultiheadDiffAttnKernel
    q1, q2, k1, k2, v, dy = (t.cuda() for t in make_inputs(1, 1, 128, 32, seed=9))
    q1.requires_grad_(True)
    lam = torch.tensor([0.5], dtype=torch.float16, device="cuda")
    y = MultiheadDiffAttnKernel(q1, q2, k1, k2, v, lam, 0.8, True)
    (g,) = torch.autograd.grad(y, q1, dy, create_graph=True)
    with pytest.raises(RuntimeError):
        g.float().sum().backward()


def test_forward_without_gradients_skips_the_backward_state():
    """Under no_grad nothing is saved for a backward: the output is bit-identical and the call allocates
    only the output, not the tensors only a backward reads (u2 and the row statistics).  The allocator's
    running total of bytes handed out is compared, which frees by earlier tests' garbage cannot lower."""
    import gc
    from layers import MultiheadDiffAttnKernel
    B, H, N, D = 2, 8, 1024, 64
    q1, q2, k1, k2, v, _ = (t.cuda() if t is not None else None for t in make_inputs(B, H, N, D, seed=10, with_dy=False))
    lam = torch.tensor([0.5], dtype=torch.float16, device="cuda")
    handed_out = lambda: torch.cuda.memory_stats()["allocated_bytes.all.allocated"]

    def call(requires_grad):
        q1.requires_grad_(requires_grad)
        gc.collect(); torch.cuda.synchronize()
        base = handed_out()
        y = MultiheadDiffAttnKernel(q1, q2, k1, k2, v, lam, 0.8, True)
        torch.cuda.synchronize()
        used = handed_out() - base
        saved = [t for t in (y.grad_fn.saved_tensors if y.grad_fn is not None else ()) if t is not None]
        return y.detach().clone(), used, saved

    y_grad, mem_grad, saved_grad = call(True)
    y_plain, mem_plain, saved_plain = call(False)
    assert torch.equal(y_grad, y_plain)
    v_bytes = v.numel() * 2
    assert mem_plain <= v_bytes + (1 << 20)              # the output only
    assert mem_grad >= 2 * v_bytes                       # output + u2 (+ statistics)
    assert not saved_plain
    # inputs, y, u2, two logsumexps, rinv, lambda
    assert sum(t.shape == v.shape for t in saved_grad) >= 3 and len(saved_grad) == 11


def test_only_the_requested_gradients_are_computed():
    """With gradients asked of q1 and lambda only, the dK/dV kernel is not launched: the other inputs get no
    gradient, and the ones asked for equal those of a full backward bit for bit."""
    from layers import MultiheadDiffAttnKernel
    ins = [t.cuda() for t in make_inputs(2, 3, 384, 64, seed=12)]
    dy = ins.pop()

    def run(grad_of):
        leaves = [t.clone().requires_grad_(i in grad_of) for i, t in enumerate(ins)]
        lam = torch.tensor([0.4], dtype=torch.float16, device="cuda", requires_grad=5 in grad_of)
        MultiheadDiffAttnKernel(*leaves, lam, 0.8, True).backward(dy)
        return [t.grad for t in leaves] + [lam.grad]

    full = run({0, 1, 2, 3, 4, 5})
    part = run({0, 5})
    assert torch.equal(part[0], full[0]) and torch.equal(part[5], full[5])
    assert all(g is None for g in part[1:5])
    kv = run({3})
    assert torch.equal(kv[3], full[3]) and all(g is None for i, g in enumerate(kv) if i != 3)
