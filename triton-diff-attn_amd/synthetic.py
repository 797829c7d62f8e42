"""Seeded synthetic inputs of the benchmark configurations, shared by bench.py, benchmark.py and the tests."""
import torch


def make_inputs(B, H, N, D, seed, scale=1.0, with_dy=True):
    """fp16 tensors drawn i.i.d. N(0, scale^2) on the CPU in the fixed order q1,q2,k1,k2,v,dy (dy is N(0,1))."""
    g = torch.Generator().manual_seed(seed)
    mk = lambda d: (torch.randn(B, H, N, d, generator=g, dtype=torch.float32) * scale).to(torch.float16)
    q1, q2, k1, k2 = mk(D), mk(D), mk(D), mk(D)
    v = mk(2 * D)
    dy = (torch.randn(B, H, N, 2 * D, generator=g, dtype=torch.float32)).to(torch.float16) if with_dy else None
    return q1, q2, k1, k2, v, dy
