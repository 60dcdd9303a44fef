"""Build-time check of the large-tile GEMM kernels' machine code.

The kernels issue their matrix instructions through inline assembly, so the compiler inserts no wait
states between a matrix instruction and a later read of its accumulator.  The source guards against that
with a drain statement every accumulator passes through; this test compiles the file for gfx950 and
checks, for every instantiation, that between the first barrier of the main loop and the drain no
instruction reads or moves an accumulator register and nothing is spilled.
"""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..")
SRC = os.path.join(ROOT, "fandhe_ai_amd", "csrc", "kern_gemm_mfma.hip")
HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="hipcc not available")
def test_no_accumulator_is_read_before_the_drain():
    with tempfile.TemporaryDirectory() as tmp:
        cmd = [HIPCC, "-O3", "-std=c++17", "--offload-arch=gfx950", "-ffp-contract=off", "-Xclang", "-target-feature",
               "-Xclang", "-packed-fp32-ops", "--cuda-device-only", "-S", "-x", "hip", SRC, "-o",
               os.path.join(tmp, "k.s")]
        subprocess.run(cmd, check=True, capture_output=True, cwd=tmp)
        text = open(os.path.join(tmp, "k.s")).read()
    kernels = re.findall(r"^(_ZN2fa1k\S*gemm_mfma_big_kernel\w*):[^\n]*\n(.*?)s_endpgm", text, flags=re.S | re.M)
    assert len(kernels) >= 12, "expected every (type, width, wavefront count) instantiation"
    for name, body in kernels:
        lines = body.split("\n")
        first = next(i for i, l in enumerate(lines) if "s_barrier" in l)
        drain = next(i for i, l in enumerate(lines) if "s_nop 15" in l)
        assert drain > first, name
        loop = lines[first:drain]
        assert any("v_mfma" in l for l in loop), name
        bad = [l.strip() for l in loop if re.search(r"v_accvgpr_read|v_accvgpr_mov|scratch_", l)]
        assert not bad, "%s: accumulator touched inside the multiply loop: %s" % (name, bad[:3])
