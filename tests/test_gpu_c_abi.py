"""The C ABI used from a C++ program without PyTorch (triton-diff-attn_amd/csrc/abi_example.cpp: hipMalloc'd
buffers, its own stream): inputs go in through a file, results come back through a file and are checked
against the oracle."""
import math
import os
import struct
import subprocess

import numpy as np
import pytest
import torch

from oracle import diff_attn_oracle as orc
from util import GRAD_RTOL, Y_ATOL, max_abs, rel_to_max

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "triton-diff-attn_amd", "abi_example")
RMS, CAUSAL, BF16, PER_HEAD = 1, 2, 4, 8


def as_u16(t):
    return t.contiguous().view(torch.int16).numpy().astype(np.int16).tobytes()


@pytest.mark.parametrize("B,H,N,D,flags,token_major", [
    (2, 3, 256, 64, RMS, False),
    (1, 4, 384, 32, RMS | CAUSAL | PER_HEAD, False),
    (1, 2, 128, 128, 0, False),
    (2, 2, 256, 64, RMS | BF16, False),
    (2, 3, 256, 64, RMS, True),              # [B,N,H,C] buffers handed over through diffattn_layout
    (2, 5, 384, 32, CAUSAL, True),
    (1, 3, 128, 128, RMS, True),
])
def test_cpp_program_matches_oracle(tmp_path, B, H, N, D, flags, token_major):
    assert os.path.exists(EXE), "abi_example is not built: run python triton-diff-attn_amd/build.py"
    dt = torch.bfloat16 if flags & BF16 else torch.float16
    g = torch.Generator().manual_seed(77 + flags)
    mk = lambda d: torch.randn(B, H, N, d, generator=g).to(dt)
    q1, q2, k1, k2, v, dy = mk(D), mk(D), mk(D), mk(D), mk(2 * D), mk(2 * D)
    lam = torch.tensor([0.7 - 0.4 * h for h in range(H)] if flags & PER_HEAD else [0.5]).to(dt)
    lambda_init, sm_scale = 0.8, 1 / math.sqrt(D)
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        f.write(struct.pack("<5i2f", B, H, N, D, flags, lambda_init, sm_scale))
        for t in (q1, q2, k1, k2, v, dy):
            f.write(as_u16(t.transpose(1, 2) if token_major else t))
        f.write(as_u16(lam))
    print("case", B, H, N, D, flags, flush=True)
    run = subprocess.run([EXE, str(fin), str(fout)] + (["token-major"] if token_major else []),
                         capture_output=True, text=True, timeout=100)
    assert run.returncode == 0, run.stderr
    raw = np.fromfile(fout, dtype=np.int16)
    qk, vv = B * H * N * D, B * H * N * 2 * D
    sizes = [vv, qk, qk, qk, qk, vv, lam.numel()]
    assert raw.size == sum(sizes)
    outs, pos = [], 0
    for n in sizes:
        outs.append(torch.from_numpy(raw[pos:pos + n].copy()).view(dt))
        pos += n
    ref = orc.forward_backward(q1, q2, k1, k2, v, lam, dy, lambda_init, bool(flags & RMS), causal=bool(flags & CAUSAL))
    y_tol, g_tol = (6e-2, 8e-2) if flags & BF16 else (Y_ATOL, GRAD_RTOL)
    y = outs[0].reshape(B, N, H, 2 * D).transpose(1, 2) if token_major else outs[0].reshape(ref[0].shape)
    assert max_abs(y, ref[0]) <= y_tol
    for name, got, want in zip(("dq1", "dq2", "dk1", "dk2", "dv", "dlambda"), outs[1:], ref[1:]):
        assert rel_to_max(got.reshape(want.shape), want) <= g_tol, name
