"""Tensors beyond 2^31 elements and 4 GiB: the offsets of the late (batch, head) units do not fit in 32 bits.
The inputs are drawn on the GPU; the oracle runs on the units of the first and of the last head, which
include the very last unit of the tensors, and every output element is checked for being finite."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, max_abs, rel_to_max

pytestmark = pytest.mark.gpu

B, H, N, D = 33, 500, 1024, 128      # 16.9 M rows: q/k tensors of 2.16 G elements (4.3 GB), v-shaped ones of 8.7 GB


def test_units_beyond_four_gigabytes():
    from layers import MultiheadDiffAttnKernel
    free, _ = torch.cuda.mem_get_info()
    if free < 120 << 30:
        pytest.skip("needs 120 GiB of free GPU memory")
    assert B * H * N * D > 2 ** 31
    print("large tensors", dict(B=B, H=H, N=N, D=D), flush=True)
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(5)
    mk = lambda d: torch.randn(B, H, N, d, generator=g, device=dev, dtype=torch.float16)
    leaves = [mk(D).requires_grad_(True) for _ in range(4)] + [mk(2 * D).requires_grad_(True)]
    dy = mk(2 * D)
    lam = torch.linspace(-0.5, 0.9, H).to(torch.float16).to(dev).requires_grad_(True)      # one lambda per head
    y = MultiheadDiffAttnKernel(*leaves, lambda_scale=lam, lambda_init=0.8, rms_norm=True)
    y.backward(dy)
    torch.cuda.synchronize()
    assert torch.isfinite(y).all()
    for t in leaves:
        assert torch.isfinite(t.grad).all()
    assert torch.isfinite(lam.grad).all()

    for h in (0, H - 1):                 # units h, H + h, ..., (B-1) H + h: the last of them ends the tensors
        cpu = lambda t: t.detach()[:, h:h + 1].float().cpu().half()
        ref = orc.forward_backward(*[cpu(t) for t in leaves], lam.detach()[h:h + 1].cpu(), cpu(dy), 0.8, True)
        assert max_abs(y.detach()[:, h:h + 1], ref[0]) <= Y_ATOL, h
        for name, t, want in zip(("dq1", "dq2", "dk1", "dk2", "dv"), leaves, ref[1:6]):
            assert rel_to_max(t.grad[:, h:h + 1], want) <= GRAD_RTOL, (name, h)
        # d(lambda_h) sums B * N rows of either sign
        scale = max(ref[6].abs().max().item(), 1e-3 * ref[5].abs().max().item() * (B * N) ** 0.5)
        assert abs(lam.grad[h].item() - ref[6].item()) <= 3 * GRAD_RTOL * scale, h
