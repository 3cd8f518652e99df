"""The 4-wave kernels keep their sums in the accumulation registers a[0:255] ACROSS assembly statements
(from a tile's K loop to its compiled epilogue, or to the next tile's K loop when the epilogue is fused):
that only works while compiled code never writes those registers.  The statements clobber all of them,
so the register allocator has no reason to use them -- this test holds it to that: the device assembly of
the kernels must contain no accumulation-register write outside the generated K loops (which have none
at all since the first K step starts its sums from zero) and no scratch use in the kernels whose loops
leave the compiler enough registers."""
import os
import re
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(HERE), "tritonblas_amd", "csrc")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


KINDS = ("fp8", "e5m2", "e4e5", "e5e4", "fp4", "bf16", "f16", "i8")


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="no hipcc")
def test_compiled_code_leaves_the_accumulators_alone(tmp_path):
    # (the generated K loops must exist: the library's build writes them)
    subprocess.run(["make", "-C", CSRC, "-s"] + [f"w4_kloop_{k}.inc" for k in KINDS] + [f"w4_clobbers_{k}.inc" for k in KINDS], check=True)
    # the two translation units of the 4-wave kernels, compiled side by side
    jobs = []
    for name in ("gemm_inst_w4", "gemm_inst_w4f8"):
        out = tmp_path / (name + ".s")
        cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-unused-command-line-argument", "-Wno-pass-failed", "-Wno-inline-asm", "-S", "--cuda-device-only",
               os.path.join(CSRC, name + ".hip"), "-o", str(out)]
        jobs.append((out, subprocess.Popen(cmd, cwd=CSRC, stderr=subprocess.DEVNULL)))
    for out, proc in jobs:
        assert proc.wait() == 0
        text = out.read_text()
        kernels = re.findall(r"^(_ZN2tb14gemm_kernel_w4\S+):", text, re.M)
        assert len(kernels) == 8     # four element types per file, each with and without the Stream-K tail
        assert "v_accvgpr_write" not in text and "v_accvgpr_mov" not in text
        # every accumulator read is one of ours: inside the generated loops (plain register names) or an
        # acc_read<N>() statement of the compiled epilogues (bracketed index)
        for line in text.splitlines():
            if "v_accvgpr_read" in line:
                assert re.search(r"v_accvgpr_read_b32 v\d+, a(\d+|\[\w+\])\s*$", line), line
        # MFMA instructions only come from the generated loops: all write a[...] and read v[...]
        mfma = [l for l in text.splitlines() if l.strip().startswith("v_mfma")]
        assert mfma and all(re.match(r"\s*v_mfma\S+ a\[\d+:\d+\], v\[\d+:\d+\], v\[\d+:\d+\], (0|a\[\d+:\d+\])", l) for l in mfma)
