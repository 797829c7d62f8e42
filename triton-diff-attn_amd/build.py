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
# the kernel sources are compiled with per-kernel resource remarks, which check_resources() reads
REMARKS = ["-Rpass-analysis=kernel-resource-usage"]
# Flags of single sources.  A kernel sized for one wave per SIMD may use 512 registers, and for such a kernel the
# compiler selects every MFMA in the form whose C and D operands are AGPRs, so each score that the VALU reads
# next costs a copy (and each reference value a copy the other way): the D = 128 forward issued two such copies
# per matrix product.  In the VGPR form its loop needs 268 registers and no copies (1.83 -> 1.75 ms at B2 H32
# N4096).  Not for the backward source, whose dK/dV kernels place their operands by hand.
SOURCE_FLAGS = {"fwd.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def check_resources(src, remarks):
    """Fails the build when a kernel that must not spill uses scratch memory.

    The dK/dV kernels issue some of their matrix products as inline assembly, for which the compiler places no
    wait states: a spilled operand reloaded (scratch_load, or v_accvgpr_write of a parked copy) directly in
    front of such a product would be read too early, silently.  The register budgets are sized by hand so
    that nothing spills; this holds the build to it.  Backward kernels: none may use scratch.  Forward
    kernels: those without dropout (last template argument) may not.
    """
    import re
    bad = []
    for name, scratch in re.findall(r"Function Name: (\S+).*?ScratchSize \[bytes/lane\]: (\d+)", remarks, re.S):
        if int(scratch) == 0:
            continue
        m = re.search(r"fwd_kernelILi\d+ELb\dELi\dELb(\d)", name)       # <D, RMS, MASK, DROP, ...>
        dropout = bool(m) and m.group(1) == "1"
        if "bwd_" in name or ("fwd_kernel" in name and not dropout):
            bad.append("%s: %s bytes of scratch per lane" % (name, scratch))
    if bad:
        raise RuntimeError("%s: kernels that must not spill do:\n  %s" % (src, "\n  ".join(bad)))


def build(verbose=True):
    objs = []
    procs = []
    # the kernel sources are compiled twice: for fp16 tensors and, with -DDA_BF16, for bf16 tensors
    units = [(src, [], src.replace(".hip", ".o")) for src in SOURCES]
    units += [(src, ["-DDA_BF16"], src.replace(".hip", "_bf16.o")) for src in KERNEL_SOURCES]
    for src, extra, obj_name in units:
        obj = os.path.join(CSRC, obj_name)
        remarks = REMARKS if src in KERNEL_SOURCES else []
        cmd = [HIPCC, *FLAGS, *SOURCE_FLAGS.get(src, []), *remarks, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, cmd, pr in procs:
        out, _ = pr.communicate()
        if pr.returncode != 0:
            out = "\n".join(l for l in out.splitlines() if "is not a recognized feature" not in l and "remark:" not in l)
            raise RuntimeError("hipcc failed: %s\n%s" % (" ".join(cmd), out))
        if src in KERNEL_SOURCES:
            check_resources(src, out)
        out = "\n".join(l for l in out.splitlines() if "is not a recognized feature" not in l and "remark:" not in l)
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
