"""The reference's own acceptance check, on the GPU: the fused kernel against the materialised PyTorch
line and the fused-library line, outputs and gradients within an absolute 1e-2 on N(0, 0.5^2) inputs
(src/kernel.py:624-635, src/benchmark.py:293-316), run through the sweep script's helper."""
import importlib.util
import os

import pytest
import torch

pytestmark = pytest.mark.gpu


def _sweep():
    path = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "triton-diff-attn_amd", "benchmark.py")
    spec = importlib.util.spec_from_file_location("sweep_benchmark", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("rms", [True, False])
@pytest.mark.parametrize("line", ["DA (PyTorch)", "DA (SDPA)"])
def test_kernel_matches_comparison_lines(line, rms):
    mod = _sweep()
    means, worst = mod.difference(mod.LINES[line][0], mod.LINES["DA (Kernel)"][0], 4, 16, 32, 256, "fwd+bwd", rms,
                                  torch.device("cuda:0"), seed=3)
    assert len(means) == 4 and worst <= 1e-2


def test_sweep_point_runs_and_reports_quantiles():
    mod = _sweep()
    rows = mod.sweep_runtime(["DA (SDPA)", "DA (Kernel)"], [512], 16, 32, "fwd+bwd", True, torch.device("cuda:0"), 0)
    r = rows[0]
    assert r["seq_len"] == 512
    for name in ("DA (SDPA)", "DA (Kernel)"):
        assert 0 < r[name + "-min"] <= r[name] <= r[name + "-max"]
    mem = mod.sweep_memory(["DA (PyTorch)", "DA (Kernel)"], [512], 16, 32, "fwd+bwd", True, torch.device("cuda:0"), 0)
    # the materialised line holds N x N score matrices, the kernel does not
    assert mem[0]["DA (Kernel)"] < mem[0]["DA (PyTorch)"]
