"""The allocation-free backward entry point, diffattn_backward_static (its workspace is a fixed array inside
the library), against diffattn_backward with a caller workspace: same results bit for bit, on two calls in
a row of which the second is the smaller problem, and a clear error beyond the array's size."""
import math

import pytest
import torch

from util import make_inputs

pytestmark = pytest.mark.gpu


def run_both(lib, native, B, H, N, D, seed, flags):
    dev = torch.device("cuda:0")
    q1, q2, k1, k2, v, dy = (t.to(dev) for t in make_inputs(B, H, N, D, seed))
    lam = torch.tensor([0.5], dtype=torch.float16, device=dev)
    y, u2 = torch.empty_like(v), torch.empty_like(v)
    lse1, lse2, rinv = (torch.empty(B, H, N, device=dev) for _ in range(3))
    stream = torch.cuda.current_stream().cuda_stream
    sm = 1 / math.sqrt(D)
    native.check(lib.diffattn_forward(q1.data_ptr(), q2.data_ptr(), k1.data_ptr(), k2.data_ptr(), v.data_ptr(),
                                      lam.data_ptr(), y.data_ptr(), u2.data_ptr(), lse1.data_ptr(), lse2.data_ptr(),
                                      rinv.data_ptr(), B, H, N, D, sm, 0.8, flags, stream))
    ins = [t.data_ptr() for t in (q1, q2, k1, k2, v, lam, y, u2, lse1, lse2, rinv, dy)]
    outs = lambda: [torch.full_like(t, float("nan")) for t in (q1, q2, k1, k2, v)] + [torch.full((1,), float("nan"), dtype=torch.float16, device=dev)]
    want, got = outs(), outs()
    ws_bytes = lib.diffattn_backward_workspace_bytes(B, H, N, D, flags)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    native.check(lib.diffattn_backward(*ins, *[t.data_ptr() for t in want], ws.data_ptr(), ws_bytes,
                                       B, H, N, D, sm, 0.8, flags, stream))
    print("static call", dict(B=B, H=H, N=N, D=D, flags=flags), flush=True)
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    native.check(lib.diffattn_backward_static(*ins, *[t.data_ptr() for t in got], B, H, N, D, sm, 0.8, flags, stream))
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    torch.cuda.synchronize()
    for name, a, b in zip(("dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), got, want):
        assert torch.isfinite(a).all(), name
        assert torch.equal(a, b), name


def test_static_scratch_backward_matches_workspace_backward():
    import _native
    lib = _native.lib()
    run_both(lib, _native, 2, 4, 1024, 64, seed=61, flags=1)      # 8192 rows
    run_both(lib, _native, 1, 3, 256, 64, seed=62, flags=1)       # a smaller problem over the same array
    run_both(lib, _native, 1, 2, 384, 128, seed=63, flags=2)      # other head dim, causal, no rms_norm
    # beyond the array: rejected before anything is launched
    p = torch.empty(16, dtype=torch.uint8, device="cuda:0").data_ptr() & ~255
    args = [p] * 18 + [4, 32, 2048, 64, 0.125, 0.8, 1, None]
    assert lib.diffattn_backward_static(*args) == -7
    assert b"scratch" in lib.diffattn_strerror(-7)
