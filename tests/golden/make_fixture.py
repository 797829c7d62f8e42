"""Writes tests/golden/diffattn_b1h2n128d32.npz: seeded fp16 inputs and the fp32 oracle's outputs.

The reference repository holds no stored vectors for this path (its only checks are two GPU-only
allclose calls, src/kernel.py:624-635 and src/benchmark.py:293-316), so this fixture comes from the
repo's own oracle after it passed tests/test_oracle.py.  It freezes the oracle's numbers: a later
edit of the oracle or of the kernels that changes results shows up against it.

Run from the repo root:  python tests/golden/make_fixture.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import diff_attn_oracle as orc  # noqa: E402
from util import make_inputs  # noqa: E402

CASES = {
    "rms": dict(lam=0.5, lambda_init=0.8, rms=True),
    "plain": dict(lam=-0.25, lambda_init=0.8, rms=False),
}


def main():
    q1, q2, k1, k2, v, dy = make_inputs(1, 2, 128, 32, seed=1234)
    out = {n: t.numpy() for n, t in zip(("q1", "q2", "k1", "k2", "v", "dy"), (q1, q2, k1, k2, v, dy))}
    for name, c in CASES.items():
        lam = torch.tensor([c["lam"]], dtype=torch.float16)
        res = orc.forward_backward(q1, q2, k1, k2, v, lam, dy, c["lambda_init"], c["rms"])
        for key, t in zip(("y", "dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), res):
            out["%s_%s" % (name, key)] = t.numpy().astype(np.float32)
        out["%s_params" % name] = np.array([c["lam"], c["lambda_init"], float(c["rms"])], dtype=np.float64)
    np.savez_compressed(os.path.join(HERE, "diffattn_b1h2n128d32.npz"), **out)


if __name__ == "__main__":
    main()
