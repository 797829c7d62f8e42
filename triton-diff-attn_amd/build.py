"""Builds libdiffattn.so (the gfx950 kernels plus their C ABI) in-tree with plain hipcc.

Usage: python build.py            (from anywhere; output lands next to this file)
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libdiffattn.so")
ABI_EXAMPLE = os.path.join(HERE, "abi_example")
SOURCES = ["fwd.hip", "bwd.hip", "api.hip"]
KERNEL_SOURCES = ["fwd.hip", "bwd.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-fp32 VALU instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fno-honor-nans",
    "-Wno-unused-command-line-argument",
]


def build(verbose=True):
    objs = []
    procs = []
    # the kernel sources are compiled twice: for fp16 tensors and, with -DDA_BF16, for bf16 tensors
    units = [(src, [], src.replace(".hip", ".o")) for src in SOURCES]
    units += [(src, ["-DDA_BF16"], src.replace(".hip", "_bf16.o")) for src in KERNEL_SOURCES]
    for src, extra, obj_name in units:
        obj = os.path.join(CSRC, obj_name)
        cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for cmd, pr in procs:
        out, _ = pr.communicate()
        out = "\n".join(l for l in out.splitlines() if "is not a recognized feature" not in l)
        if pr.returncode != 0:
            raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
        if verbose and out.strip():
            print(out)
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    # the C++ example of the C ABI (also driven by a GPU test): links the library, no PyTorch
    cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", os.path.join(CSRC, "abi_example.cpp"),
           "-L" + HERE, "-ldiffattn", "-Wl,-rpath,$ORIGIN", "-o", ABI_EXAMPLE]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    return LIB


if __name__ == "__main__":
    build()
    print("built", LIB)
    sys.exit(0)
