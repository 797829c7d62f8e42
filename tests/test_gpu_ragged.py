"""Sequence lengths that are not multiples of 128 (a restriction of the reference's kernels, which have no
boundary checks, src/kernel.py:4, :136-150, :527): the kernels run on the next multiple of 128, never touch a
row of the caller's tensors past the real length, and ignore the padding keys; nothing is padded or copied on
the host.  Checked against the fp32 oracle at the real length, with the tolerances of the other parity tests."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("N,D,rms,causal", [
    (1, 64, False, False),       # a single token: X = (1 - lambda) v
    (37, 64, True, False),
    (100, 32, False, False),
    (129, 64, True, False),      # one real row in the second block
    (200, 128, True, False),
    (333, 64, False, True),
    (450, 128, True, True),
    (1000, 64, True, False),
    (1000, 32, True, True),
])
def test_ragged_lengths_match_oracle(N, D, rms, causal):
    q1, q2, k1, k2, v, dy = make_inputs(1, 2, N, D, seed=31)
    y, grads = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, rms, dy, causal=causal)
    assert y.shape == v.shape and all(g.shape == t.shape for g, t in zip(grads[:5], (q1, q2, k1, k2, v)))
    ref = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([0.5], dtype=torch.float16), dy, 0.8, rms, chunk=1,
                               causal=causal)
    assert max_abs(y, ref[0]) <= Y_ATOL
    for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), grads, ref[1:]):
        if r.abs().max().item() < 1e-6:      # e.g. one token: the softmax of a single key has no gradient
            assert g.float().abs().max().item() <= 2e-3, name
        else:
            assert rel_to_max(g, r) <= GRAD_RTOL, name


@pytest.mark.parametrize("N", [1, 2, 3, 70])
@pytest.mark.parametrize("rms", [True, False])
def test_short_sequences_with_large_scores(N, rms):
    """With few real keys and scores of magnitude ~10 a row's logsumexp is often far below zero, so
    exp(0 - lse) of a padding key is huge: the backward must mask padding keys, not rely on their zero rows."""
    q1, q2, k1, k2, v, dy = make_inputs(4, 8, N, 32, seed=34, scale=3.0)
    y, grads = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, rms, dy)
    ref = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([0.5], dtype=torch.float16), dy, 0.8, rms, chunk=1)
    assert torch.isfinite(y).all() and max_abs(y, ref[0]) <= 3 * Y_ATOL      # |v| is three times the usual
    for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), grads, ref[1:]):
        assert torch.isfinite(g).all(), name
        # a single key has no softmax gradient and, with rms_norm, no d(lambda): what is left is the
        # rounding noise of operands three times the usual size
        tol = GRAD_RTOL * r.abs().max().item() if r.abs().max().item() >= 1e-3 else 2e-2
        assert max_abs(g, r) <= tol, name


def test_single_token_closed_form():
    q1, q2, k1, k2, v, _ = make_inputs(2, 3, 1, 64, seed=32)
    y, _ = run_kernel(q1, q2, k1, k2, v, 0.25, 0.8, False)
    assert max_abs(y, 0.75 * v.float()) <= 2e-3


def test_padding_does_not_leak_into_real_rows():
    # the result for 200 rows must not depend on what a caller stores behind them
    q1, q2, k1, k2, v, dy = make_inputs(1, 2, 256, 64, seed=33)
    cut = [t[:, :, :200].contiguous() for t in (q1, q2, k1, k2, v)]
    y_a, g_a = run_kernel(*cut, 0.5, 0.8, True, dy[:, :, :200].contiguous())
    views = [t[:, :, :200] for t in (q1, q2, k1, k2, v)]                  # non-contiguous views of longer tensors
    y_b, g_b = run_kernel(*views, 0.5, 0.8, True, dy[:, :, :200])
    assert torch.equal(y_a, y_b) and all(torch.equal(a, b) for a, b in zip(g_a, g_b))


@pytest.mark.parametrize("D,n_valid,causal,rms", [(64, 200, False, True), (32, 130, True, True), (128, 255, False, False),
                                                   (64, 70, True, False), (64, 129, False, True)])
def test_rows_past_the_real_length_are_neither_read_nor_written(D, n_valid, causal, rms):
    """Through the C ABI, on buffers of the padded length: input rows past n_valid hold NaN (a kernel that read
    them would spread it), output rows past n_valid hold a sentinel (a kernel that wrote them would erase it)."""
    import math
    import _native
    lib = _native.lib()
    B, H, N = 2, 3, 256
    cpu = make_inputs(B, H, N, D, seed=35)
    dev = [t.cuda() for t in cpu]
    for t in dev:
        t[:, :, n_valid:] = float("nan")
    q1, q2, k1, k2, v, dy = dev
    lam = torch.tensor([0.5], dtype=torch.float16, device="cuda")
    sentinel = 777.0
    y = torch.full_like(v, sentinel)
    u2 = torch.empty_like(v)
    lse1, lse2, rinv = (torch.empty(B, H, N, device="cuda") for _ in range(3))
    grads = [torch.full_like(t, sentinel) for t in (q1, q2, k1, k2, v)]
    dlam = torch.empty(1, dtype=torch.float16, device="cuda")
    flags = (1 if rms else 0) | (2 if causal else 0)
    ws_bytes = lib.diffattn_backward_workspace_bytes(B, H, N, D, flags)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    sm = 1 / math.sqrt(D)
    _native.check(lib.diffattn_forward_padded(q1.data_ptr(), q2.data_ptr(), k1.data_ptr(), k2.data_ptr(), v.data_ptr(),
                                              lam.data_ptr(), y.data_ptr(), u2.data_ptr(), lse1.data_ptr(), lse2.data_ptr(),
                                              rinv.data_ptr(), B, H, N, n_valid, D, sm, 0.8, flags, None, None, st))
    _native.check(lib.diffattn_backward_stages(q1.data_ptr(), q2.data_ptr(), k1.data_ptr(), k2.data_ptr(), v.data_ptr(),
                                               lam.data_ptr(), y.data_ptr(), u2.data_ptr(), lse1.data_ptr(), lse2.data_ptr(),
                                               rinv.data_ptr(), dy.data_ptr(), *[g.data_ptr() for g in grads], dlam.data_ptr(),
                                               ws.data_ptr(), ws_bytes, B, H, N, n_valid, D, sm, 0.8, flags, 15, None, None, st))
    torch.cuda.synchronize()
    cut = [t[:, :, :n_valid].contiguous() for t in cpu]
    ref = orc.forward_backward(*cut[:5], torch.tensor([0.5], dtype=torch.float16), cut[5], 0.8, rms, chunk=1, causal=causal)
    assert (y[:, :, n_valid:] == sentinel).all() and all((g[:, :, n_valid:] == sentinel).all() for g in grads)
    assert max_abs(y[:, :, :n_valid], ref[0]) <= Y_ATOL
    for name, g, r in zip(("dq1", "dq2", "dk1", "dk2", "dv"), grads, ref[1:6]):
        assert torch.isfinite(g[:, :, :n_valid]).all(), name
        assert rel_to_max(g[:, :, :n_valid], r) <= GRAD_RTOL, name
    assert rel_to_max(dlam, ref[6]) <= GRAD_RTOL


def test_nothing_is_copied_for_a_ragged_length():
    """The operator hands the caller's tensors to the kernels as they are: the output and the gradients have the
    real length, and the gradients of token-major views come back in that layout."""
    from layers import MultiheadDiffAttnKernel
    B, H, N, D = 2, 4, 200, 64
    cpu = make_inputs(B, H, N, D, seed=36)
    # [B,N,H,.] buffers seen as [B,H,N,.]
    leaves = [t.cuda().transpose(1, 2).contiguous().transpose(1, 2).requires_grad_(True) for t in cpu[:5]]
    lam = torch.tensor([0.5], dtype=torch.float16, device="cuda", requires_grad=True)
    y = MultiheadDiffAttnKernel(*leaves, lambda_scale=lam, lambda_init=0.8, rms_norm=True)
    assert y.shape == (B, H, N, 2 * D) and y.stride() == leaves[4].stride()
    y.backward(cpu[5].cuda())
    torch.cuda.synchronize()
    assert all(t.grad.shape == t.shape and t.grad.stride() == t.stride() for t in leaves)
    ref = orc.forward_backward(*cpu[:5], torch.tensor([0.5], dtype=torch.float16), cpu[5], 0.8, True, chunk=1)
    assert max_abs(y, ref[0]) <= Y_ATOL
    for name, t, r in zip(("dq1", "dq2", "dk1", "dk2", "dv"), leaves, ref[1:6]):
        assert rel_to_max(t.grad, r) <= GRAD_RTOL, name
