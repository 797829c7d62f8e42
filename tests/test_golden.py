"""Committed fixture (tests/golden/diffattn_b1h2n128d32.npz) against the oracle (CPU) and the kernels (GPU)."""
import os

import numpy as np
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, max_abs, rel_to_max, run_kernel

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "diffattn_b1h2n128d32.npz")
KEYS = ("y", "dq1", "dq2", "dk1", "dk2", "dv", "dlambda")


def load():
    z = np.load(FIX)
    ins = [torch.from_numpy(z[n]) for n in ("q1", "q2", "k1", "k2", "v", "dy")]
    return z, ins


@pytest.mark.parametrize("case", ["rms", "plain"])
def test_oracle_reproduces_fixture(case):
    z, (q1, q2, k1, k2, v, dy) = load()
    lam, li, rms = z[case + "_params"]
    res = orc.forward_backward(q1, q2, k1, k2, v, torch.tensor([lam], dtype=torch.float16), dy, float(li), bool(rms))
    for key, t in zip(KEYS, res):
        ref = torch.from_numpy(z["%s_%s" % (case, key)])
        assert torch.allclose(t, ref, rtol=1e-4, atol=1e-5), key


@pytest.mark.gpu
@pytest.mark.parametrize("case", ["rms", "plain"])
def test_kernels_match_fixture(case):
    z, (q1, q2, k1, k2, v, dy) = load()
    lam, li, rms = z[case + "_params"]
    y, grads = run_kernel(q1, q2, k1, k2, v, float(lam), float(li), bool(rms), dy)
    assert max_abs(y, torch.from_numpy(z[case + "_y"])) <= Y_ATOL
    for key, g in zip(KEYS[1:], grads):
        assert rel_to_max(g, torch.from_numpy(z["%s_%s" % (case, key)])) <= GRAD_RTOL, key
