"""Shared helpers of the parity tests: seeded synthetic inputs and the tolerance metrics."""
import torch

from synthetic import make_inputs  # noqa: F401  (the benchmark draws the same tensors)

# tolerances stated by the build's target: outputs within max-abs 2e-2 of the fp32 oracle,
# gradients within 5e-2 relative to the max-norm of the oracle gradient
Y_ATOL = 2e-2
GRAD_RTOL = 5e-2


def max_abs(a, b):
    return (a.float().cpu() - b.float().cpu()).abs().max().item()


def rel_to_max(a, ref):
    ref = ref.float().cpu()
    return (a.float().cpu() - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)


def run_kernel(q1, q2, k1, k2, v, lam_value, lambda_init, rms_norm, dy=None, device="cuda", causal=False):
    """Runs layers.MultiheadDiffAttnKernel on the GPU; returns (y, grads or None) as CPU tensors."""
    from layers import MultiheadDiffAttnKernel

    need = dy is not None
    t = [x.to(device).requires_grad_(need) for x in (q1, q2, k1, k2, v)]
    # one lambda, or a list with one per head
    lam = torch.tensor(list(lam_value) if isinstance(lam_value, (list, tuple)) else [lam_value],
                       dtype=q1.dtype, device=device, requires_grad=need)
    extra = {"causal": True} if causal else {}
    y = MultiheadDiffAttnKernel(*t, lambda_scale=lam, lambda_init=lambda_init, rms_norm=rms_norm, **extra)
    grads = None
    if need:
        y.backward(dy.to(device))
        grads = [x.grad.cpu() for x in t] + [lam.grad.cpu()]
    torch.cuda.synchronize()
    return y.detach().cpu(), grads
