"""The stock-PyTorch comparison lines of the sweep (baselines.py) against the fp32 oracle, on the CPU,
and the host-side helpers of the sweep script.  The reference's own check between its PyTorch line
and its kernel is an absolute 1e-2 (src/benchmark.py:293); the same bound is used here for the
fp16 comparison lines against the oracle."""
import importlib.util
import os

import pytest
import torch

import baselines
from oracle import diff_attn_oracle as orc
from util import make_inputs, max_abs

ATOL = 1e-2


def _case(seed=5, B=1, H=2, N=64, D=16):
    q1, q2, k1, k2, v, _ = make_inputs(B, H, N, D, seed, 0.5)
    return q1, q2, k1, k2, v


@pytest.mark.parametrize("rms", [False, True])
@pytest.mark.parametrize("fn", [baselines.MultiheadDiffAttn, baselines.MultiheadFlashDiffAttn])
def test_differential_lines_follow_the_oracle(fn, rms):
    q1, q2, k1, k2, v = _case()
    lam = torch.tensor([0.4], dtype=torch.float16)
    ref = orc.forward(q1, q2, k1, k2, v, lam, 0.8, rms)[0]
    got = fn(q1, q2, k1, k2, v, lambda_scale=lam, lambda_init=0.8, rms_norm=rms)
    assert got.dtype == torch.float16 and got.shape == v.shape
    assert max_abs(got.float(), ref) <= ATOL


def test_lambda_may_be_a_python_float():
    q1, q2, k1, k2, v = _case()
    a = baselines.MultiheadDiffAttn(q1, q2, k1, k2, v, lambda_scale=0.5, rms_norm=True)
    b = baselines.MultiheadDiffAttn(q1, q2, k1, k2, v, lambda_scale=torch.tensor([0.5], dtype=torch.float16), rms_norm=True)
    assert max_abs(a.float(), b.float()) <= 2e-3


@pytest.mark.parametrize("rms", [False, True])
def test_plain_lines_agree_with_each_other_and_with_lambda_zero(rms):
    q1, q2, k1, k2, v = _case()
    q = torch.cat([q1, q2], -1)
    k = torch.cat([k1, k2], -1)
    a = baselines.MultiheadAttn(q, k, v, rms_norm=rms)
    b = baselines.MultiheadFlashAttn(q, k, v, rms_norm=rms)
    assert max_abs(a.float(), b.float()) <= ATOL
    # lambda = 0 turns the differential operator into plain attention of stream 1 (no (1-lambda_init) factor without the norm)
    if not rms:
        d = baselines.MultiheadDiffAttn(q1, q2, k1, k2, v, lambda_scale=0.0)
        assert max_abs(d.float(), baselines.MultiheadAttn(q1, k1, v).float()) <= 2e-3


def test_gradients_of_the_materialised_line_follow_the_oracle():
    q1, q2, k1, k2, v = _case(N=32)
    dy = torch.randn(v.shape, generator=torch.Generator().manual_seed(1)).half()
    lam = torch.tensor([0.4], dtype=torch.float16)
    ref = orc.forward_backward(q1, q2, k1, k2, v, lam, dy, 0.8, True, chunk=1)
    leaves = [t.clone().requires_grad_(True) for t in (q1, q2, k1, k2, v)]
    lam_leaf = lam.clone().requires_grad_(True)
    baselines.MultiheadDiffAttn(*leaves, lambda_scale=lam_leaf, lambda_init=0.8, rms_norm=True).backward(dy)
    for t, r in zip(leaves, ref[1:6]):
        assert max_abs(t.grad.float(), r) <= 5e-2 * r.abs().max().item() + 1e-3


def _load_sweep_module():
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "triton-diff-attn_amd", "benchmark.py")
    spec = importlib.util.spec_from_file_location("sweep_benchmark", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_sweep_script_host_helpers():
    mod = _load_sweep_module()
    assert mod.quantile([1.0, 2.0, 3.0, 4.0, 5.0], 0.5) == 3.0
    assert mod.quantile([1.0, 2.0], 0.05) == pytest.approx(1.05)
    assert set(mod.LINES) == {"A (PyTorch)", "A (SDPA)", "DA (PyTorch)", "DA (SDPA)", "DA (Kernel)"}
    assert all(mod.TOKENS % n == 0 for n in mod.SEQ_LENS)
    gen = torch.Generator().manual_seed(0)
    args, kwargs, dout = mod.make_case(True, 2, 3, 16, 8, gen, "cpu")
    assert [tuple(a.shape) for a in args] == [(2, 3, 16, 8)] * 4 + [(2, 3, 16, 16)]
    assert kwargs["lambda_scale"].shape == (1,) and dout.shape == args[-1].shape
    assert all(a.requires_grad and a.dtype == torch.float16 for a in args)
    args, kwargs, _ = mod.make_case(False, 2, 3, 16, 8, gen, "cpu")
    assert [tuple(a.shape) for a in args] == [(2, 3, 16, 16)] * 3 and kwargs == {}


@pytest.mark.parametrize("fn", [baselines.MultiheadDiffAttn, baselines.MultiheadFlashDiffAttn])
def test_causal_comparison_lines_follow_the_oracle(fn):
    q1, q2, k1, k2, v = _case()
    lam = torch.tensor([0.4], dtype=torch.float16)
    ref = orc.forward(q1, q2, k1, k2, v, lam, 0.8, True, causal=True)
    got = fn(q1, q2, k1, k2, v, lambda_scale=lam, lambda_init=0.8, rms_norm=True, causal=True)
    assert max_abs(got.float(), ref) <= ATOL
