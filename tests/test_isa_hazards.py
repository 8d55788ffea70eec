"""The Q6_K GEMM epilogue reads its activation scale through hand-written `v_fmac_f32_dpp` instructions
(inline assembly, so the compiler's hazard recogniser does not see them).  CDNA requires two wait states
between a VALU write of a register and a DPP read of it: compile the kernel to assembly and check that
no VALU instruction writes the DPP source register within the two instructions before each use."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


@pytest.mark.skipif(not os.path.exists(HIPCC) and not shutil.which("hipcc"), reason="hipcc not available")
def test_no_valu_write_right_before_a_dpp_read(tmp_path):
    out = tmp_path / "gemm.s"
    cmd = [HIPCC if os.path.exists(HIPCC) else "hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only", os.path.join(ROOT, "strix.rs_amd", "csrc", "gemm.hip"), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True, timeout=600)
    lines = [l.strip() for l in out.read_text().splitlines()]
    lines = [l for l in lines if l and not l.startswith((";", ".")) and not l.endswith(":")]
    uses = 0
    for i, l in enumerate(lines):
        m = re.match(r"v_fmac_f32_dpp (v\d+), (v\d+), (v\d+)", l)
        if not m:
            continue
        uses += 1
        src = m.group(2)
        for k in (1, 2):
            p = lines[i - k]
            if not p.startswith("v_") or p.startswith("v_fmac_f32_dpp"):
                continue
            dst = p.split()[1].rstrip(",")
            r = re.match(r"v\[(\d+):(\d+)\]", dst)
            written = [dst] if not r else [f"v{n}" for n in range(int(r.group(1)), int(r.group(2)) + 1)]
            assert src not in written, f"`{p}` writes {src} {k} instruction(s) before `{l}`"
    assert uses >= 16      # the kernel still has its broadcast multiply-adds
