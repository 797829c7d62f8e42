"""Compiles the backward kernels to gfx950 assembly (no GPU needed) and checks that no inline-assembly
MFMA reads a register that a VALU instruction wrote immediately before it (see isa_scan.py)."""
import os
import shutil
import subprocess

import pytest

import isa_scan

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "triton-diff-attn_amd", "csrc")


def test_scanner_flags_a_write_right_before_an_asm_mfma():
    bad = """
\tv_accvgpr_write_b32 a67, v137
\t;;#ASMSTART
\tv_mfma_f32_32x32x16_f16 v[18:33], v[66:69], a[64:67], v[18:33]
\t;;#ASMEND
"""
    assert len(isa_scan.asm_mfma_hazards(bad)) == 1
    spaced = bad.replace("\t;;#ASMSTART", "\ts_nop 2\n\t;;#ASMSTART")
    assert isa_scan.asm_mfma_hazards(spaced) == []
    # a compiler-visible MFMA is the compiler's business; an LDS load is ordered by s_waitcnt
    assert isa_scan.asm_mfma_hazards(bad.replace("\t;;#ASMSTART\n", "").replace("\t;;#ASMEND\n", "")) == []
    assert isa_scan.asm_mfma_hazards(bad.replace("v_accvgpr_write_b32 a67, v137", "ds_read_b128 v[66:69], v1")) == []
    assert isa_scan.registers("v[2:4], a7, s[0:1], v10") == {"v2", "v3", "v4", "a7", "v10"}


def _load_build():
    import importlib.util
    spec = importlib.util.spec_from_file_location("da_build", os.path.join(ROOT, "triton-diff-attn_amd", "build.py"))
    build = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(build)
    return build


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    """Assembly text of the three compilations the tests below read (backward fp16 and bf16, forward fp16),
    compiled side by side."""
    build = _load_build()
    tmp = tmp_path_factory.mktemp("isa")
    jobs = {}
    for key, src, variant in (("bwd_fp16", "bwd.hip", []), ("bwd_bf16", "bwd.hip", ["-DDA_BF16"]), ("fwd_fp16", "fwd.hip", [])):
        out = tmp / (key + ".s")
        cmd = [build.HIPCC] + [f for f in build.FLAGS if f != "-fPIC"] + build.SOURCE_FLAGS.get(src, []) + variant + ["--cuda-device-only", "-S", "-o", str(out),
                                                                              os.path.join(CSRC, src)]
        jobs[key] = (out, subprocess.Popen(cmd, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE))
    texts = {}
    for key, (out, proc) in jobs.items():
        _, err = proc.communicate()
        assert proc.returncode == 0, err.decode()[-2000:]
        texts[key] = out.read_text()
    return texts


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
@pytest.mark.parametrize("variant", ["fp16", "bf16"])
def test_backward_kernels_have_no_unprotected_asm_mfma(assembly, variant):
    text = assembly["bwd_" + variant]
    variant = variant == "bf16"
    assert ("v_mfma_f32_32x32x16_bf16" if variant else "v_mfma_f32_32x32x16_f16") in text and ";;#ASMSTART" in text
    hazards = isa_scan.asm_mfma_hazards(text)
    assert hazards == [], "VALU write right before an inline-asm MFMA: %s" % hazards[:5]
    # the build switches the packed-fp32 VALU instructions off; none may appear in the generated code
    import re
    packed = re.findall(r"^\s*(v_pk_(?:fma|mul|add)_f32)\b", text, re.M)
    assert packed == [], "packed fp32 instructions in the backward kernels: %d" % len(packed)
    # nothing spills: the kernels' register budgets are sized by hand, and spill code inside the
    # software-pipelined loops has produced wrong results on the GPU
    assert "scratch_" not in text, "a backward kernel uses scratch memory"


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc")
def test_forward_kernels_do_not_spill_in_their_loops(assembly):
    """The forward instantiations without dropout use no scratch memory at all; those with dropout may
    park a value across the main loop, but never inside it."""
    import re
    kernels = re.findall(r"^(_Z\w*fwd_kernel\w*):[^\n]*\n(.*?)s_endpgm", assembly["fwd_fp16"], re.S | re.M)
    # D <= 64: rms_norm x mask x dropout in 128-row workgroups plus the 64-row variants of the plain ones (14 each);
    # D = 128: rms_norm x mask x dropout in 64-row workgroups plus the 128-row variants of the plain ones (14)
    assert len(kernels) == 42
    for name, body in kernels:
        dropout = re.search(r"fwd_kernelILi\d+ELb\dELi\dELb(\d)", name).group(1) == "1"
        if not dropout:
            assert "scratch_" not in body, name
            continue
        # inside a loop = between a loop header label and the backward branch to it
        lines = body.split("\n")
        label_at = {m.group(1): i for i, l in enumerate(lines) if (m := re.match(r"^(\.LBB\w+):", l))}
        for i, l in enumerate(lines):
            m = re.match(r"\s+s_cbranch_\w+ (\.LBB\w+)", l)
            if m and label_at.get(m.group(1), i) < i:
                assert not any("scratch_" in x for x in lines[label_at[m.group(1)]:i]), name


def test_build_rejects_a_spilling_kernel():
    """build.py reads the compiler's per-kernel resource remarks and refuses kernels that must not spill."""
    build = _load_build()
    remark = ("x.hip:1:1: remark: Function Name: %s [-Rpass-analysis=kernel-resource-usage]\n"
              "x.hip:1:1: remark:     VGPRs: 256 [-Rpass-analysis=kernel-resource-usage]\n"
              "x.hip:1:1: remark:     ScratchSize [bytes/lane]: %d [-Rpass-analysis=kernel-resource-usage]\n")
    dkdv = "_ZN2da15bwd_dkdv_kernelILi64ELi0ELb0ELb0EEEvN6da_abi10BwdParamsTIDF16_EE"
    fwd_plain = "_ZN2da10fwd_kernelILi64ELb1ELi0ELb0ELb1EEEvN6da_abi10FwdParamsTIDF16_EE"
    fwd_drop = "_ZN2da10fwd_kernelILi64ELb1ELi1ELb1ELb0EEEvN6da_abi10FwdParamsTIDF16_EE"
    build.check_resources("x.hip", remark % (dkdv, 0) + remark % (fwd_plain, 0) + remark % (fwd_drop, 24))
    for name in (dkdv, fwd_plain):
        with pytest.raises(RuntimeError, match="must not spill"):
            build.check_resources("x.hip", remark % (dkdv, 0) + remark % (name, 16))
