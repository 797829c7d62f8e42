"""One lambda per head (a tensor of H values instead of one; not in the reference): GPU parity against
the oracle, which is pinned for this case head by head against its single-lambda form."""
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, make_inputs, max_abs, rel_to_max, run_kernel

pytestmark = pytest.mark.gpu

CASES = [
    # B, H, N, D, rms, causal
    (2, 4, 256, 64, True, False),
    (3, 5, 384, 32, False, False),    # odd head count, N not a multiple of 256
    (1, 3, 256, 128, True, False),
    (2, 4, 200, 64, True, True),      # padded and causal
]


@pytest.mark.parametrize("B,H,N,D,rms,causal", CASES)
def test_per_head_lambda_matches_oracle(B, H, N, D, rms, causal):
    q1, q2, k1, k2, v, dy = make_inputs(B, H, N, D, seed=31)
    lams = [0.8 - 0.35 * h for h in range(H)]              # positive, zero-ish and negative values
    lam16 = torch.tensor(lams, dtype=torch.float16)
    print("case", B, H, N, D, rms, causal, flush=True)
    y, grads = run_kernel(q1, q2, k1, k2, v, lams, 0.8, rms, dy=dy, causal=causal)
    ref = orc.forward_backward(q1, q2, k1, k2, v, lam16, dy, 0.8, rms, causal=causal)
    assert max_abs(y, ref[0]) <= Y_ATOL
    for name, got, want in zip(("dq1", "dq2", "dk1", "dk2", "dv"), grads[:5], ref[1:6]):
        assert rel_to_max(got, want) <= GRAD_RTOL, name
    assert grads[5].shape == (H,)
    assert rel_to_max(grads[5], ref[6]) <= GRAD_RTOL


def test_equal_lambdas_give_the_single_lambda_result_bit_for_bit():
    B, H, N, D = 2, 4, 256, 64
    q1, q2, k1, k2, v, dy = make_inputs(B, H, N, D, seed=32)
    y1, g1 = run_kernel(q1, q2, k1, k2, v, 0.5, 0.8, True, dy=dy)
    yh, gh = run_kernel(q1, q2, k1, k2, v, [0.5] * H, 0.8, True, dy=dy)
    assert torch.equal(y1, yh)
    for a, b in zip(g1[:5], gh[:5]):
        assert torch.equal(a, b)
    # the single d(lambda) is the sum of the per-head ones, up to their fp16 rounding
    assert abs(g1[5].float().item() - gh[5].float().sum().item()) <= 4e-3 * max(1.0, abs(g1[5].float().item()))


@pytest.mark.parametrize("per_head", [False, True])
@pytest.mark.parametrize("D", [32, 128])
def test_dlambda_is_the_same_whichever_launch_sums_it(D, per_head):
    """The fixed-order sum of the d(lambda) partials runs in extra workgroups of the dK/dV launch, of the dQ
    launch when there is no dK/dV launch, and as a kernel of its own when there is neither: bit-identical."""
    import math

    import _native
    from util import make_inputs
    lib = _native.lib()
    B, H, N = 3, 5, 384
    dev = torch.device("cuda:0")
    flags = 1 | (8 if per_head else 0)
    q1, q2, k1, k2, v, dy = (t.to(dev) for t in make_inputs(B, H, N, D, seed=71))
    lam = torch.linspace(-0.4, 0.9, H if per_head else 1).to(torch.float16).to(dev)
    y, u2 = torch.empty_like(v), torch.empty_like(v)
    lse1, lse2, rinv = (torch.empty(B, H, N, device=dev) for _ in range(3))
    stream = torch.cuda.current_stream().cuda_stream
    sm = 1 / math.sqrt(D)
    _native.check(lib.diffattn_forward(q1.data_ptr(), q2.data_ptr(), k1.data_ptr(), k2.data_ptr(), v.data_ptr(),
                                       lam.data_ptr(), y.data_ptr(), u2.data_ptr(), lse1.data_ptr(), lse2.data_ptr(),
                                       rinv.data_ptr(), B, H, N, D, sm, 0.8, flags, stream))
    ins = [t.data_ptr() for t in (q1, q2, k1, k2, v, lam, y, u2, lse1, lse2, rinv, dy)]
    ws_bytes = lib.diffattn_backward_workspace_bytes(B, H, N, D, flags)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    results = []
    for masks in ((15,), (1, 2 | 4), (1, 2 | 8), (1, 2), (1 | 4 | 8, 2)):
        grads = [torch.full_like(t, float("nan")) for t in (q1, q2, k1, k2, v)]
        dlam = torch.full((lam.numel(),), float("nan"), dtype=torch.float16, device=dev)
        for mask in masks:
            print("stages", mask, dict(D=D, per_head=per_head), flush=True)
            _native.check(lib.diffattn_backward_stages(*ins, *[g.data_ptr() for g in grads], dlam.data_ptr(),
                                                       ws.data_ptr(), ws_bytes, B, H, N, N, D, sm, 0.8, flags, mask,
                                                       None, None, stream))
        torch.cuda.synchronize()
        assert torch.isfinite(dlam).all(), masks
        results.append((dlam, grads))
    for dlam, _ in results[1:]:
        assert torch.equal(dlam, results[0][0])
    # the hosting launches still write all of their own results
    for a, b in zip(results[0][1], results[4][1]):
        assert torch.equal(a, b)
    assert torch.equal(results[1][1][2], results[0][1][2]) and torch.equal(results[2][1][0], results[0][1][0])
