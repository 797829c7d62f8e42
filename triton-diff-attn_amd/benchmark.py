#!/usr/bin/env python3
"""Sequence-length sweep: run time, peak memory and output difference of the fused differential
attention against stock-PyTorch lines, on one GPU.

Follows the shape of the reference's sweep (src/benchmark.py:19-25, 53-148, 181-250, 253-345):
sequence lengths 512 .. 16384 at batch = 16384 / seq_len, 16 heads, head dim 32 (v has 64),
fp16, N(0, 0.5^2) inputs, uniform upstream gradient, a random 1-element lambda on the device;
"fwd" or "fwd+bwd"; median / 5 % / 95 % quantiles of the run time.  Lines:

  A (PyTorch)   A (SDPA)   DA (PyTorch)   DA (SDPA)   DA (Kernel)

"SDPA" is torch's fused attention, standing in for the flash-attn wheel of the reference, which
does not exist for this GPU.  Timing uses device events around each call instead of
triton.testing.do_bench.  Results go to <out>/{runtime,memory,difference}.csv and to stdout.

  python benchmark.py --mode fwd+bwd --out results/MI355X_backward_16_32_RMS_norm
"""
import argparse
import csv
import math
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from baselines import MultiheadAttn, MultiheadDiffAttn, MultiheadFlashAttn, MultiheadFlashDiffAttn  # noqa: E402
from layers import MultiheadDiffAttnKernel  # noqa: E402

LINES = {
    "A (PyTorch)": (MultiheadAttn, False),
    "A (SDPA)": (MultiheadFlashAttn, False),
    "DA (PyTorch)": (MultiheadDiffAttn, True),
    "DA (SDPA)": (MultiheadFlashDiffAttn, True),
    "DA (Kernel)": (MultiheadDiffAttnKernel, True),
}
SEQ_LENS = [512, 1024, 2048, 4096, 8192, 16384]
TOKENS = 16384          # batch * seq_len of every point of the sweep


def make_case(differential, batch, heads, seq_len, head_dim, gen, device):
    """Leaf tensors of one sweep point, drawn like the reference's harness (src/benchmark.py:43-50, 118-126)."""
    def leaf(*shape):
        x = torch.empty(*shape, dtype=torch.float16, device=device).normal_(0.0, 0.5, generator=gen)
        return x.requires_grad_(True)

    if differential:
        args = [leaf(batch, heads, seq_len, head_dim) for _ in range(4)] + [leaf(batch, heads, seq_len, 2 * head_dim)]
        kwargs = {"lambda_scale": leaf(1)}
    else:
        args = [leaf(batch, heads, seq_len, 2 * head_dim) for _ in range(3)]
        kwargs = {}
    dout = torch.rand(args[-1].shape, dtype=torch.float16, device=device, generator=gen)
    return args, kwargs, dout


def call(fn, args, kwargs, dout, mode, rms_norm):
    for t in list(args) + list(kwargs.values()):
        t.grad = None
    y = fn(*args, rms_norm=rms_norm, **kwargs)
    if mode == "fwd+bwd":
        y.backward(dout)
    return y


def quantile(sorted_vals, q):
    pos = q * (len(sorted_vals) - 1)
    lo, hi = int(math.floor(pos)), int(math.ceil(pos))
    return sorted_vals[lo] + (sorted_vals[hi] - sorted_vals[lo]) * (pos - lo)


def time_call(run, target_ms=200.0, min_rep=10, max_rep=200):
    """Median, 5 % and 95 % quantile (ms) of `run`, one event pair per call."""
    for _ in range(3):
        run()
    torch.cuda.synchronize()
    probe0, probe1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    probe0.record(); run(); probe1.record()
    torch.cuda.synchronize()
    reps = int(max(min_rep, min(max_rep, target_ms / max(probe0.elapsed_time(probe1), 1e-3))))
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in pairs:
        a.record(); run(); b.record()
    torch.cuda.synchronize()
    ms = sorted(a.elapsed_time(b) for a, b in pairs)
    return quantile(ms, 0.5), quantile(ms, 0.05), quantile(ms, 0.95)


def sweep_runtime(lines, seq_lens, heads, head_dim, mode, rms_norm, device, seed):
    rows = []
    for n in seq_lens:
        row = {"seq_len": n}
        for name in lines:
            fn, differential = LINES[name]
            gen = torch.Generator(device=device).manual_seed(seed)
            try:
                args, kwargs, dout = make_case(differential, TOKENS // n, heads, n, head_dim, gen, device)
                med, lo, hi = time_call(lambda: call(fn, args, kwargs, dout, mode, rms_norm))
            except RuntimeError as exc:       # out of memory for the materialised lines at long sequences
                if "out of memory" not in str(exc).lower():
                    raise
                med = lo = hi = float("nan")
            finally:
                args = kwargs = dout = None
                torch.cuda.empty_cache()
            row[name], row[name + "-min"], row[name + "-max"] = med, lo, hi
            print("runtime  N=%-6d %-14s %9.3f ms  (p5 %.3f, p95 %.3f)" % (n, name, med, lo, hi), flush=True)
        rows.append(row)
    return rows


def sweep_memory(lines, seq_lens, heads, head_dim, mode, rms_norm, device, seed):
    rows = []
    for n in seq_lens:
        row = {"seq_len": n}
        for name in lines:
            fn, differential = LINES[name]
            gen = torch.Generator(device=device).manual_seed(seed)
            try:
                args, kwargs, dout = make_case(differential, TOKENS // n, heads, n, head_dim, gen, device)
                torch.cuda.synchronize()
                torch.cuda.reset_peak_memory_stats()
                call(fn, args, kwargs, dout, mode, rms_norm)
                torch.cuda.synchronize()
                row[name] = torch.cuda.max_memory_allocated() / 2**20
            except RuntimeError as exc:
                if "out of memory" not in str(exc).lower():
                    raise
                row[name] = float("nan")
            finally:
                args = kwargs = dout = None
                torch.cuda.empty_cache()
            print("memory   N=%-6d %-14s %10.1f MiB peak" % (n, name, row[name]), flush=True)
        rows.append(row)
    return rows


def difference(fn_a, fn_b, repeats, heads, head_dim, seq_len, mode, rms_norm, device, seed, atol=1e-2):
    """Mean |y_a - y_b| over `repeats` random cases; raises if an output or a gradient differs by more than atol
    (the check of src/benchmark.py:253-345, here with the bound reported instead of asserted away)."""
    gen = torch.Generator(device=device).manual_seed(seed)
    means, worst = [], 0.0
    for _ in range(repeats):
        args, kwargs, dout = make_case(True, 1, heads, seq_len, head_dim, gen, device)
        got = []
        for fn in (fn_a, fn_b):
            y = call(fn, args, kwargs, dout, mode, rms_norm)
            grads = [t.grad.clone() for t in args] if mode == "fwd+bwd" else []
            got.append([y.detach()] + grads)
        for a, b in zip(*got):
            worst = max(worst, (a.float() - b.float()).abs().max().item())
        means.append((got[0][0].float() - got[1][0].float()).abs().mean().item())
    if worst > atol:
        raise AssertionError("outputs or gradients differ by %.3e (> %.1e)" % (worst, atol))
    return means, worst


def write_csv(path, rows):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=list(rows[0].keys()))
        w.writeheader()
        w.writerows(rows)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--mode", default="fwd+bwd", choices=["fwd", "fwd+bwd"])
    ap.add_argument("--seq-lens", type=int, nargs="+", default=SEQ_LENS)
    ap.add_argument("--num-heads", type=int, default=16)
    ap.add_argument("--head-dim", type=int, default=32, help="q/k head dim; v has twice as many features")
    ap.add_argument("--no-rms-norm", action="store_true")
    ap.add_argument("--lines", nargs="+", default=list(LINES), choices=list(LINES))
    ap.add_argument("--what", nargs="+", default=["difference", "memory", "runtime"],
                    choices=["difference", "memory", "runtime"])
    ap.add_argument("--out", default=None, help="folder for the csv files (default: none written)")
    ap.add_argument("--seed", type=int, default=0)
    args = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("benchmark.py needs a GPU")
    device = torch.device("cuda:0")
    rms = not args.no_rms_norm
    common = (args.num_heads, args.head_dim)
    if "difference" in args.what:
        means, worst = difference(MultiheadDiffAttn, MultiheadDiffAttnKernel, 20, *common, 256, args.mode, rms, device, args.seed)
        print("difference DA (PyTorch) vs DA (Kernel): mean |dy| %.3e, worst output/gradient element %.3e" %
              (sum(means) / len(means), worst), flush=True)
        if args.out:
            write_csv(os.path.join(args.out, "difference.csv"), [{"case": i, "mean_abs_diff": m} for i, m in enumerate(means)])
    if "memory" in args.what:
        rows = sweep_memory(args.lines, args.seq_lens, *common, args.mode, rms, device, args.seed)
        if args.out:
            write_csv(os.path.join(args.out, "memory.csv"), rows)
    if "runtime" in args.what:
        rows = sweep_runtime(args.lines, args.seq_lens, *common, args.mode, rms, device, args.seed)
        if args.out:
            write_csv(os.path.join(args.out, "runtime.csv"), rows)


if __name__ == "__main__":
    main()
