"""Tensors handed over through their strides (the reference passes Q1's and V's strides to its kernels,
src/kernel.py:487-494): permuted views, slices of larger buffers and a strided upstream gradient give the
oracle's results, and the same bits as dense copies of the same values, without the host copying them."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max

pytestmark = pytest.mark.gpu

NAMES = ("dq1", "dq2", "dk1", "dk2", "dv", "dlambda")


def run(tensors, dy, lam_value, lambda_init, rms, causal=False):
    from layers import MultiheadDiffAttnKernel
    leaves = [t.detach().requires_grad_(True) for t in tensors]
    lam = torch.tensor([lam_value], dtype=torch.float16, device="cuda", requires_grad=True)
    y = MultiheadDiffAttnKernel(*leaves, lambda_scale=lam, lambda_init=lambda_init, rms_norm=rms,
                                **({"causal": True} if causal else {}))
    y.backward(dy)
    torch.cuda.synchronize()
    return y.detach(), [t.grad for t in leaves] + [lam.grad]


def token_major(t):
    """The same values in a [B,N,H,C] buffer, viewed as [B,H,N,C]."""
    return t.transpose(1, 2).contiguous().transpose(1, 2)


@pytest.mark.parametrize("D,N,H,rms,causal", [(64, 256, 3, True, False), (32, 384, 5, False, True), (128, 128, 2, True, False),
                                                (64, 1024, 8, True, True)])
def test_token_major_views_match_oracle_and_dense(D, N, H, rms, causal):
    B = 2
    cpu = make_inputs(B, H, N, D, seed=300 + D)
    dense = [t.cuda() for t in cpu]
    print("strided case", dict(B=B, H=H, N=N, D=D, rms=rms, causal=causal), flush=True)
    views = [token_major(t) for t in dense]
    assert not views[0].is_contiguous()
    y_d, g_d = run(dense[:5], dense[5], 0.5, 0.8, rms, causal)
    y_v, g_v = run(views[:5], views[5], 0.5, 0.8, rms, causal)
    assert y_v.stride() == views[4].stride(), "the output takes v's layout: a following [B,N,H*2d] reshape is free"
    assert torch.equal(y_v, y_d)
    for name, a, b in zip(NAMES, g_v, g_d):
        assert torch.equal(a, b), name
    ref = orc.forward_backward(*cpu[:5], torch.tensor([0.5], dtype=torch.float16), cpu[5], 0.8, rms, causal=causal)
    assert max_abs(y_v, ref[0]) <= Y_ATOL
    for name, g, r in zip(NAMES, g_v, ref[1:]):
        assert rel_to_max(g, r) <= GRAD_RTOL, name


def test_slices_of_a_fused_projection_are_read_in_place():
    """q1 and q2 (k1 and k2) as the two halves of one [B,N,H,2,d] projection output, v from its own: what
    modules.DiffAttn hands over.  Base pointers differ, strides are shared, nothing is dense."""
    B, H, N, d = 2, 4, 256, 64
    g = torch.Generator().manual_seed(77)
    qproj = torch.randn(B, N, H, 2, d, generator=g).half().cuda()
    kproj = torch.randn(B, N, H, 2, d, generator=g).half().cuda()
    vproj = torch.randn(B, N, H, 2 * d, generator=g).half().cuda()
    dy = torch.randn(B, N, H, 2 * d, generator=g).half().cuda().transpose(1, 2)
    q = qproj.permute(3, 0, 2, 1, 4)
    k = kproj.permute(3, 0, 2, 1, 4)
    v = vproj.transpose(1, 2)
    views = [q[0], q[1], k[0], k[1], v]
    y_v, g_v = run(views, dy, 0.4, 0.8, True)
    y_d, g_d = run([t.contiguous() for t in views], dy.contiguous(), 0.4, 0.8, True)
    assert torch.equal(y_v, y_d)
    for name, a, b in zip(NAMES, g_v, g_d):
        assert torch.equal(a, b), name


def test_unsuitable_strides_fall_back_to_a_copy():
    """A last dimension that is not contiguous, or rows that are not 16-byte aligned, cannot be read in
    place: the host copies, the result is the same."""
    B, H, N, D = 1, 2, 128, 32
    cpu = make_inputs(B, H, N, D, seed=78)
    dense = [t.cuda() for t in cpu]
    odd = []
    for t in dense[:5]:
        wide = torch.zeros(*t.shape[:3], t.shape[3] + 4, dtype=t.dtype, device="cuda")     # row stride C + 4
        wide[..., :t.shape[3]] = t
        odd.append(wide[..., :t.shape[3]])
    y_o, g_o = run(odd, dense[5], 0.5, 0.8, True)
    y_d, g_d = run(dense[:5], dense[5], 0.5, 0.8, True)
    assert torch.equal(y_o, y_d) and all(torch.equal(a, b) for a, b in zip(g_o, g_d))
