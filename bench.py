#!/usr/bin/env python3
"""Headline benchmark: forward+backward differential attention on one MI355X.

A step is one forward + one backward of `layers.MultiheadDiffAttnKernel` at B=4, H=32, N=2048,
D=64 (fp16, rms_norm on, lambda 0.5, lambda_init 0.8) on seeded synthetic N(0,1) inputs that are
resident in HBM before the timed region.  Prints ONE JSON line.

  value       fwd+bwd TFLOP/s, algorithmic matmul FLOPs = 32*B*H*N^2*D per step
              (forward 12*B*H*N^2*D, backward 20*B*H*N^2*D; 2 FLOP per MAC, softmax not counted)
  roofline    the dominant kernel (dK/dV backward) against the fp16 dense MFMA peak, timed with
              events on the launch stream
  cpu_baseline  the fp32 oracle (forward + autograd backward) on a few (batch, head) units of the
              same workload on the host cores, scaled to the same FLOP count
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "triton-diff-attn_amd"))

PEAK_FP16_TFLOPS = 2500.0     # MI355X published dense fp16 MFMA peak (2.5 PFLOP/s)

WORKLOADS = {
    "headline": dict(B=4, H=32, N=2048, D=64, lam=0.5, lambda_init=0.8, rms=True, seed=2, scale=1.0),
    "config1": dict(B=2, H=16, N=512, D=32, lam=0.5, lambda_init=0.8, rms=True, seed=0, scale=1.0),
    "config4": dict(B=8, H=32, N=4096, D=128, lam=0.8, lambda_init=0.2, rms=False, seed=4, scale=1.0),
    # the headline shape with the causal mask (an addition to the reference's operator)
    "headline_causal": dict(B=4, H=32, N=2048, D=64, lam=0.5, lambda_init=0.8, rms=True, seed=2, scale=1.0, causal=True),
    # the operator's additions to the reference, at the headline shape: what each costs against "headline"
    "headline_bf16": dict(B=4, H=32, N=2048, D=64, lam=0.5, lambda_init=0.8, rms=True, seed=2, scale=1.0, bf16=True),
    "headline_dropout": dict(B=4, H=32, N=2048, D=64, lam=0.5, lambda_init=0.8, rms=True, seed=2, scale=1.0, dropout=0.1),
    "headline_per_head": dict(B=4, H=32, N=2048, D=64, lam=0.5, lambda_init=0.8, rms=True, seed=2, scale=1.0, per_head=True),
    # q/k/v as views of token-major [B,N,H,.] buffers (a projection's output), read through their strides
    "headline_token_major": dict(B=4, H=32, N=2048, D=64, lam=0.5, lambda_init=0.8, rms=True, seed=2, scale=1.0, token_major=True),
    # a sequence length that is not a multiple of the kernels' 128-row blocks
    "headline_ragged": dict(B=4, H=32, N=2000, D=64, lam=0.5, lambda_init=0.8, rms=True, seed=2, scale=1.0),
    # forward-only configurations: a step is one forward without gradients
    "config0": dict(B=2, H=16, N=512, D=32, lam=0.5, lambda_init=0.8, rms=True, seed=0, scale=1.0, fwd_only=True),
    "headline_fwd": dict(B=4, H=32, N=2048, D=64, lam=0.5, lambda_init=0.8, rms=True, seed=2, scale=1.0, fwd_only=True),
    "config3": dict(B=1, H=16, N=16384, D=64, lam=0.3, lambda_init=0.8, rms=True, seed=3, scale=0.5, fwd_only=True),
    "config3_no_norm": dict(B=1, H=16, N=16384, D=64, lam=0.3, lambda_init=0.8, rms=False, seed=3, scale=0.5, fwd_only=True),
}


def flops(cfg):
    """Algorithmic matmul FLOPs (forward, backward); with the causal mask only the N(N+1)/2 visible
    (query, key) pairs count."""
    pairs = cfg["N"] * (cfg["N"] + 1) // 2 if cfg.get("causal") else cfg["N"] ** 2
    unit = cfg["B"] * cfg["H"] * pairs * cfg["D"]
    return 12 * unit, 20 * unit


def event_time(fn, iters, torch, each=None):
    """Average milliseconds per call of fn over `iters` calls, measured with events on the current stream.
    With a list in `each`, an event is also recorded between calls and the per-call times are appended to it."""
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(iters + 1 if each is not None else 2)]
    torch.cuda.synchronize()
    marks[0].record()
    for i in range(iters):
        fn()
        if each is not None:
            marks[i + 1].record()
    if each is None:
        marks[1].record()
    torch.cuda.synchronize()
    if each is not None:
        each.extend(a.elapsed_time(b) for a, b in zip(marks[:-1], marks[1:]))
    return marks[0].elapsed_time(marks[-1]) / iters


def quantile(values, q):
    """Linear-interpolation quantile of a list (what the reference's do_bench reports, src/benchmark.py:94)."""
    v = sorted(values)
    pos = q * (len(v) - 1)
    lo = int(pos)
    hi = min(lo + 1, len(v) - 1)
    return v[lo] + (v[hi] - v[lo]) * (pos - lo)


def gpu_max_clock_mhz(torch):
    """Maximum engine clock of GPU 0 in MHz, from the device properties or, failing that, rocminfo."""
    mhz = getattr(torch.cuda.get_device_properties(0), "clock_rate", 0) / 1e3
    if mhz > 0:
        return mhz
    try:
        import re
        import subprocess
        text = subprocess.run(["rocminfo"], capture_output=True, text=True, timeout=30).stdout
        # agents are listed in order; take the first one whose device type is GPU
        for agent in text.split("*******")[1:]:
            if re.search(r"Device Type:\s+GPU", agent):
                m = re.search(r"Max Clock Freq\. \(MHz\):\s+(\d+)", agent)
                if m:
                    return float(m.group(1))
    except Exception:
        pass
    return None


def cpu_baseline(cfg, torch, budget_s=12.0):
    """Times the fp32 oracle (forward + autograd backward) on a few (b,h) units of the workload."""
    from oracle import diff_attn_oracle as orc
    from synthetic import make_inputs

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    N, D = cfg["N"], cfg["D"]
    units = 8 if N <= 4096 else 2
    q1, q2, k1, k2, v, dy = make_inputs(1, units, N, D, cfg["seed"], cfg["scale"])
    lam = torch.tensor([cfg["lam"]], dtype=torch.float16)
    if cfg.get("fwd_only"):
        run = lambda: orc.forward(q1, q2, k1, k2, v, lam, cfg["lambda_init"], cfg["rms"], chunk=1)
    else:
        run = lambda: orc.forward_backward(q1, q2, k1, k2, v, lam, dy, cfg["lambda_init"], cfg["rms"], chunk=1,
                                           causal=bool(cfg.get("causal")))
    run()  # warm-up
    t0 = time.perf_counter()
    reps = 0
    while True:
        run()
        reps += 1
        if time.perf_counter() - t0 > budget_s or reps >= 200:
            break
    dt = (time.perf_counter() - t0) / reps
    f_fwd, f_bwd = flops(dict(cfg, B=1, H=units))
    fl = float(f_fwd if cfg.get("fwd_only") else f_fwd + f_bwd)
    return {
        "value": fl / dt / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": "%d of %d (batch,head) units of the workload, fp32 oracle %s, %d repetitions, "
                  "%.3f s per repetition" % (units, cfg["B"] * cfg["H"],
                                             "forward" if cfg.get("fwd_only") else "forward+autograd backward", reps, dt),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--workload", default="headline", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--graph", action="store_true",
                    help="capture the whole step in one HIP graph (torch.cuda.CUDAGraph) and time its replays: what a "
                         "small problem costs once Python, the autograd engine and the allocator are out of the way")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch
    import _native
    from layers import MultiheadDiffAttnKernel
    from synthetic import make_inputs

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    cfg = WORKLOADS[args.workload]
    B, H, N, D = cfg["B"], cfg["H"], cfg["N"], cfg["D"]
    dev = torch.device("cuda:0")
    prop = torch.cuda.get_device_properties(0)
    lib = _native.lib()

    dtype = torch.bfloat16 if cfg.get("bf16") else torch.float16
    q1, q2, k1, k2, v, dy = (t.to(dev).to(dtype) for t in make_inputs(B, H, N, D, cfg["seed"], cfg["scale"]))
    if cfg.get("token_major"):
        # the same values in [B,N,H,.] memory, seen as [B,H,N,.]
        q1, q2, k1, k2, v = (t.transpose(1, 2).contiguous().transpose(1, 2) for t in (q1, q2, k1, k2, v))
    fwd_only = bool(cfg.get("fwd_only"))
    leaves = [t.requires_grad_(not fwd_only) for t in (q1, q2, k1, k2, v)]
    lam = torch.tensor([cfg["lam"]] * (H if cfg.get("per_head") else 1), dtype=dtype, device=dev, requires_grad=not fwd_only)
    extra = {}
    if cfg.get("causal"):
        extra["causal"] = True
    if cfg.get("dropout"):
        extra.update(dropout_p=cfg["dropout"], dropout_seed=1234)

    def step():
        if fwd_only:
            with torch.no_grad():
                MultiheadDiffAttnKernel(*leaves, lambda_scale=lam, lambda_init=cfg["lambda_init"], rms_norm=cfg["rms"], **extra)
            return
        for t in leaves:
            t.grad = None
        lam.grad = None
        y = MultiheadDiffAttnKernel(*leaves, lambda_scale=lam, lambda_init=cfg["lambda_init"], rms_norm=cfg["rms"], **extra)
        y.backward(dy)

    if args.graph:
        # the whole step (forward, backward, gradient assignment) captured once and replayed: no Python,
        # no autograd engine and no allocator in the timed region
        eager_step = step
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                eager_step()
        torch.cuda.current_stream().wait_stream(side)
        for t in leaves:
            t.grad = None
        lam.grad = None
        whole = torch.cuda.CUDAGraph()
        with torch.cuda.graph(whole):
            if fwd_only:
                with torch.no_grad():
                    MultiheadDiffAttnKernel(*leaves, lambda_scale=lam, lambda_init=cfg["lambda_init"], rms_norm=cfg["rms"], **extra)
            else:
                MultiheadDiffAttnKernel(*leaves, lambda_scale=lam, lambda_init=cfg["lambda_init"], rms_norm=cfg["rms"],
                                        **extra).backward(dy)

        def step():      # noqa: F811  (replaces the eager step)
            whole.replay()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    per_step = []
    t0 = time.perf_counter()
    ms_events = event_time(step, args.steps, torch, each=per_step)
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    ms_per_step = max(ms_events, wall_ms)

    f_fwd, f_bwd = flops(cfg)
    f_step = f_fwd if fwd_only else f_fwd + f_bwd
    value = f_step / (ms_per_step * 1e-3) / 1e12

    # ---- per-kernel timings through the C ABI, events on the launch stream ----
    with torch.no_grad():
        n_pad = -(-N // 128) * 128
        # a length that is not a multiple of 128 runs on the next one inside the kernels; only the library's own
        # buffers (u2, the row statistics, the workspace) have the padded length
        kq1, kq2, kk1, kk2, kv, kdy = q1, q2, k1, k2, v, dy
        yb = torch.empty_like(kv); u2 = torch.empty(B, H, n_pad, 2 * D, device=dev, dtype=dtype)
        lse1 = torch.empty(B, H, n_pad, device=dev); lse2 = torch.empty(B, H, n_pad, device=dev)
        rinv = torch.empty(B, H, n_pad, device=dev)
        grads = [torch.empty_like(t) for t in (kq1, kq2, kk1, kk2, kv)]      # in the layout of their tensors
        dlam = torch.empty(lam.numel(), dtype=dtype, device=dev)
        # DIFFATTN_RMS_NORM | DIFFATTN_CAUSAL | DIFFATTN_BF16 | DIFFATTN_LAMBDA_PER_HEAD | DIFFATTN_UNPADDED
        flags = (int(cfg["rms"]) | (2 if cfg.get("causal") else 0) | (4 if cfg.get("bf16") else 0)
                 | (8 if cfg.get("per_head") else 0) | (32 if n_pad != N else 0))
        layout = None
        if cfg.get("token_major"):
            layout = _native.Layout(*kq1.stride()[:3], *kv.stride()[:3], *yb.stride()[:3], *kdy.stride()[:3],
                                    *grads[0].stride()[:3], *grads[4].stride()[:3])
        drop = _native.Dropout(cfg["dropout"], 1234) if cfg.get("dropout") else None
        ws_bytes = lib.diffattn_backward_workspace_bytes(B, H, n_pad, D, flags)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        stream = torch.cuda.current_stream().cuda_stream
        sm = 1 / math.sqrt(D)

        def launch_forward():
            _native.check(lib.diffattn_forward_padded(
                kq1.data_ptr(), kq2.data_ptr(), kk1.data_ptr(), kk2.data_ptr(), kv.data_ptr(), lam.data_ptr(),
                yb.data_ptr(), u2.data_ptr(), lse1.data_ptr(), lse2.data_ptr(), rinv.data_ptr(),
                B, H, n_pad, N, D, sm, cfg["lambda_init"], flags, layout, drop, stream))

        def bwd_stage(mask):
            return lambda: _native.check(lib.diffattn_backward_stages(
                kq1.data_ptr(), kq2.data_ptr(), kk1.data_ptr(), kk2.data_ptr(), kv.data_ptr(), lam.data_ptr(),
                yb.data_ptr(), u2.data_ptr(), lse1.data_ptr(), lse2.data_ptr(), rinv.data_ptr(), kdy.data_ptr(),
                *[g.data_ptr() for g in grads], dlam.data_ptr(), ws.data_ptr(), ws_bytes,
                B, H, n_pad, N, D, sm, cfg["lambda_init"], flags, mask, layout, drop, stream))

        k_iters = max(5, min(args.steps, 30))
        for _ in range(3):          # the buffers above are new: first touches stay out of the timings
            launch_forward()
        kernels_ms = {"fwd_kernel": event_time(launch_forward, k_iters, torch)}
        if not fwd_only:
            for _ in range(3):
                bwd_stage(15)()
            # the fixed-order sum of the d(lambda) partials rides in the dK/dV launch of a full backward
            kernels_ms.update({
                "bwd_prep_kernel": event_time(bwd_stage(1), k_iters, torch),
                "bwd_dkdv_kernel": event_time(bwd_stage(4), k_iters, torch),
                "bwd_dq_kernel": event_time(bwd_stage(8), k_iters, torch),
            })
    unit = f_fwd // 12
    # the dominant kernel: dK/dV backward, S1,S2 (4) + dP (4) + dV (4) + dK1,dK2 (4), times B*H*N^2*D;
    # in a forward-only workload the forward kernel with its 12*B*H*N^2*D
    dom, dom_flops = ("fwd_kernel", 12 * unit) if fwd_only else ("bwd_dkdv_kernel", 16 * unit)
    dom_tflops = dom_flops / (kernels_ms[dom] * 1e-3) / 1e12
    # HBM bytes per launch are not measured in this run: they are read from the committed summary of two
    # rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) of this workload, when there is one (see the file's note)
    traffic = traffic_source = None
    tpath = os.path.join(ROOT, "profiles", "traffic_%s.json" % args.workload)
    if os.path.exists(tpath):
        k = json.load(open(tpath))["kernels"].get(dom)
        if k:
            traffic = k["fetch_bytes"] + k["write_bytes"]
            traffic_source = "profiles/traffic_%s.json (static: rocprofv3 --pmc summary, not measured in this run)" % args.workload
    roofline = {
        "bound": "mfma", "kernel": dom, "achieved": dom_tflops, "peak": PEAK_FP16_TFLOPS,
        "unit": "TFLOP/s", "frac": dom_tflops / PEAK_FP16_TFLOPS, "traffic": traffic,
        "traffic_source": traffic_source, "flops_per_launch": dom_flops, "ms_per_launch": kernels_ms[dom],
    }

    out = {
        "metric": "fwd+bwd TFLOP/s & % fp16 MFMA peak, diff-attn B4 H32 N2048 D64",
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if cfg.get("bf16") else "f16", "data": "synthetic",
        "config": {"workload": "%s: diff-attn %s B%d H%d N%d D%d rms_norm=%s lambda=%.1f lambda_init=%.1f"
                               % (args.workload, "fwd" if fwd_only else "fwd+bwd", B, H, N, D, cfg["rms"], cfg["lam"],
                                  cfg["lambda_init"])
                               + (" causal" if cfg.get("causal") else "") + (" bf16" if cfg.get("bf16") else "")
                               + (" dropout=%.2f" % cfg["dropout"] if cfg.get("dropout") else "")
                               + (" one lambda per head" if cfg.get("per_head") else "")
                               + (" token-major q/k/v read through strides" if cfg.get("token_major") else "")
                               + (" (HIP graph replay)" if args.graph else "")},
        "frac_of_fp16_mfma_peak": value / PEAK_FP16_TFLOPS,
        # the K timed steps one by one (an event between steps): median and the 5 % / 95 % quantiles
        "ms_per_step_median": quantile(per_step, 0.5), "ms_per_step_p5": quantile(per_step, 0.05),
        "ms_per_step_p95": quantile(per_step, 0.95),
        "value_at_median": f_step / (quantile(per_step, 0.5) * 1e-3) / 1e12,
        "fwd_tflops": f_fwd / (kernels_ms["fwd_kernel"] * 1e-3) / 1e12,
        "bwd_tflops": None if fwd_only else
        f_bwd / (sum(kernels_ms[k] for k in kernels_ms if k.startswith("bwd")) * 1e-3) / 1e12,
        "kernels_ms": kernels_ms,
        "device": {"name": prop.name, "cus": prop.multi_processor_count,
                   "clock_mhz": gpu_max_clock_mhz(torch), "peak_fp16_tflops_used": PEAK_FP16_TFLOPS},
        "roofline": roofline,
    }
    if args.workload != "headline":
        out["metric"] = "%s TFLOP/s & %% fp16 MFMA peak, diff-attn" % ("fwd" if fwd_only else "fwd+bwd")
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, torch)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
