"""Dropout on the two softmax maps (a feature the reference lists as missing, src/kernel.py:4).  The kernels
regenerate their keep decisions from a hash of (seed, stream, unit, query, key); the library writes the same
decisions out (diffattn_dropout_mask), and the fp32 oracle is run with exactly those masks."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max

pytestmark = pytest.mark.gpu

NAMES = ("dq1", "dq2", "dk1", "dk2", "dv", "dlambda")


def kernel_masks(B, H, n_pad, p, seed):
    """The keep decisions of both softmax maps as bool [B,H,n_pad,n_pad] CPU tensors."""
    import _native
    lib = _native.lib()
    cfg = _native.Dropout(p, seed)
    out = []
    for stream in (0, 1):
        keep = torch.empty(B, H, n_pad, n_pad, dtype=torch.uint8, device="cuda")
        _native.check(lib.diffattn_dropout_mask(keep.data_ptr(), B, H, n_pad, stream, cfg, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        out.append(keep.cpu().bool())
    return out


def run(cpu, lam_value, lambda_init, rms, causal, p, seed):
    from layers import MultiheadDiffAttnKernel
    leaves = [t.cuda().requires_grad_(True) for t in cpu[:5]]
    lam = torch.tensor([lam_value], dtype=torch.float16, device="cuda", requires_grad=True)
    y = MultiheadDiffAttnKernel(*leaves, lambda_scale=lam, lambda_init=lambda_init, rms_norm=rms, causal=causal,
                                dropout_p=p, dropout_seed=seed)
    y.backward(cpu[5].cuda())
    torch.cuda.synchronize()
    return y.detach().cpu(), [t.grad.cpu() for t in leaves] + [lam.grad.cpu()]


@pytest.mark.parametrize("D,N,p,rms,causal", [
    (64, 256, 0.1, True, False),
    (64, 384, 0.5, False, False),
    (32, 256, 0.1, True, True),
    (32, 128, 0.5, True, False),
    (128, 128, 0.1, False, False),
    (128, 256, 0.5, True, True),
    (64, 200, 0.25, True, False),       # padded sequence: the masks are indexed with the padded length
])
def test_dropout_matches_oracle_with_the_kernels_masks(D, N, p, rms, causal):
    B, H, seed = 2, 3, 1234 + D + N
    cpu = make_inputs(B, H, N, D, seed=400 + D)
    print("dropout case", dict(B=B, H=H, N=N, D=D, p=p, rms=rms, causal=causal), flush=True)
    n_pad = -(-N // 128) * 128
    m1, m2 = (m[:, :, :N, :N] for m in kernel_masks(B, H, n_pad, p, seed))
    p_eff = round(p * 256) / 256
    frac = m1.float().mean().item()
    assert abs(frac - (1 - p_eff)) < 0.01, "keep fraction %.4f" % frac
    assert (m1 != m2).any(), "the two maps draw independent masks"
    y, grads = run(cpu, 0.5, 0.8, rms, causal, p, seed)
    ref = orc.forward_backward(*cpu[:5], torch.tensor([0.5], dtype=torch.float16), cpu[5], 0.8, rms, causal=causal,
                               keep1=m1, keep2=m2, dropout_p=p_eff)
    assert torch.isfinite(y).all()
    assert max_abs(y, ref[0]) <= Y_ATOL
    for name, g, r in zip(NAMES, grads, ref[1:]):
        assert torch.isfinite(g).all(), name
        assert rel_to_max(g, r) <= GRAD_RTOL, name


def test_dropout_is_a_function_of_the_seed():
    cpu = make_inputs(1, 2, 256, 64, seed=41)
    a = run(cpu, 0.5, 0.8, True, False, 0.2, 7)
    b = run(cpu, 0.5, 0.8, True, False, 0.2, 7)
    c = run(cpu, 0.5, 0.8, True, False, 0.2, 8)
    assert torch.equal(a[0], b[0]) and all(torch.equal(x, z) for x, z in zip(a[1], b[1]))
    assert not torch.equal(a[0], c[0])


def test_zero_probability_is_the_plain_operator():
    from layers import MultiheadDiffAttnKernel
    q1, q2, k1, k2, v, _ = (t.cuda() for t in make_inputs(1, 2, 128, 32, seed=42))
    lam = torch.tensor([0.5], dtype=torch.float16, device="cuda")
    plain = MultiheadDiffAttnKernel(q1, q2, k1, k2, v, lam, 0.8, True)
    zero = MultiheadDiffAttnKernel(q1, q2, k1, k2, v, lam, 0.8, True, dropout_p=0.0, dropout_seed=5)
    assert torch.equal(plain, zero)
    with pytest.raises(ValueError):
        MultiheadDiffAttnKernel(q1, q2, k1, k2, v, lam, 0.8, True, dropout_p=1.0)


def test_mask_dump_equals_the_host_model_of_the_hash():
    """Bit for bit: the library's keep decisions against tests/dropout_model.py, whose statistics the CPU
    tests check (keep rate, independence across seeds, units and streams)."""
    import numpy as np
    import dropout_model as dm
    B, H, N, p = 2, 3, 128, 0.25
    for seed in (0, 1, 0x1234_5678_9ABC_DEF0):
        m1, m2 = kernel_masks(B, H, N, p, seed)
        for unit in (0, 1, B * H - 1):
            b, h = divmod(unit, H)
            assert np.array_equal(m1[b, h].numpy(), dm.keep_mask(seed, unit, 0, N, p)), (seed, unit, 0)
            assert np.array_equal(m2[b, h].numpy(), dm.keep_mask(seed, unit, 1, N, p)), (seed, unit, 1)


def test_dropout_under_stream_capture_needs_a_seed():
    from layers import MultiheadDiffAttnKernel
    cpu = make_inputs(1, 2, 128, 64, seed=5)
    t = [x.cuda() for x in cpu[:5]]
    lam = torch.tensor([0.5], dtype=torch.float16, device="cuda")
    MultiheadDiffAttnKernel(*t, lambda_scale=lam, dropout_p=0.1)       # eager: a seed is drawn
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        MultiheadDiffAttnKernel(*t, lambda_scale=lam, dropout_p=0.1, dropout_seed=3)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        with pytest.raises(RuntimeError, match="explicit dropout_seed"):
            MultiheadDiffAttnKernel(*t, lambda_scale=lam, dropout_p=0.1)
        y = MultiheadDiffAttnKernel(*t, lambda_scale=lam, dropout_p=0.1, dropout_seed=3)     # a named seed is fine
    g.replay()
    torch.cuda.synchronize()
    assert torch.isfinite(y).all()
