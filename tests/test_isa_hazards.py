"""The Q6_K GEMM epilogue, the small-batch kernel and the grouped MoE GEMM read their activation scale through hand-written
`v_fmac_f32_dpp` instructions (inline assembly, so the compiler's hazard recogniser does not see them).  CDNA requires two
wait states between a VALU write of a register and a DPP read of it: compile every source file that holds such an
instruction to assembly and check that no VALU instruction writes the DPP source register within the two instructions
before each use."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _dpp_sources():
    """Source files of the library with a hand-written DPP multiply-add."""
    csrc = os.path.join(ROOT, "strix.rs_amd", "csrc")
    headers = [n for n in os.listdir(csrc) if n.endswith(".h") and "v_fmac_f32_dpp" in open(os.path.join(csrc, n)).read()]
    names = []
    for n in sorted(os.listdir(csrc)):
        text = open(os.path.join(csrc, n)).read() if n.endswith(".hip") else ""
        if "v_fmac_f32_dpp" in text or any(f'"{h}"' in text for h in headers):
            names.append(n)
    assert "gemm.hip" in names and "skinny.hip" in names
    return names


@pytest.mark.skipif(not os.path.exists(HIPCC) and not shutil.which("hipcc"), reason="hipcc not available")
@pytest.mark.parametrize("source", _dpp_sources())
def test_no_valu_write_right_before_a_dpp_read(tmp_path, source):
    out = tmp_path / (source + ".s")
    cmd = [HIPCC if os.path.exists(HIPCC) else "hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only", os.path.join(ROOT, "strix.rs_amd", "csrc", source), "-o", str(out)]
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


def _kernel_lines(asm, mangled_prefix):
    """Instruction lines of the first kernel whose symbol starts with `mangled_prefix`."""
    lines = asm.splitlines()
    start = next(i for i, l in enumerate(lines) if l.startswith(mangled_prefix) and l.split(";")[0].rstrip().endswith(":"))
    out = []
    for l in lines[start + 1:]:
        t = l.strip()
        if t.startswith("s_endpgm"):
            break
        if t and not t.startswith((";", ".")) and not t.endswith(":"):
            out.append(t)
    return out


@pytest.mark.skipif(not os.path.exists(HIPCC) and not shutil.which("hipcc"), reason="hipcc not available")
def test_flat_gemv_waits_for_the_activation_only(tmp_path):
    """The flat GEMV requests the activation before the weights and issues its weight loads without
    conditions, so that (a wave's loads complete in order) the quantiser waits with vmcnt = number of
    weight loads in flight, and each ring slot is consumed with an exact count.  A conditional load or a
    reordered request would silently turn these into vmcnt(0): check the compiled single-row Q4_0 kernel."""
    out = tmp_path / "gemv.s"
    cmd = [HIPCC if os.path.exists(HIPCC) else "hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "-S", "--cuda-device-only", os.path.join(ROOT, "strix.rs_amd", "csrc", "gemv.hip"), "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True, timeout=900)
    ins = _kernel_lines(out.read_text(), "_ZN3smx16gemv_flat_kernelINS_7OpsQ4_0ELi1ELi3ELi16ELi1ELb0ELb0EEE")
    is_weight = lambda l: l.startswith(("global_load_ushort", "global_load_dwordx4 v")) and l.split()[-1] == "off"   # the activation's loads use the scalar base form
    first_weight = next(i for i, l in enumerate(ins) if is_weight(l))
    # the staging barrier: the first one behind the weight requests (a long row has the waves meet once in front of them)
    barrier = next(i for i, l in enumerate(ins) if i > first_weight and l.startswith("s_barrier"))
    loads = [i for i, l in enumerate(ins[:barrier]) if l.startswith("global_load")]
    weight_loads = [i for i in loads if is_weight(ins[i])]
    assert len(weight_loads) == 6                      # three units: 16 bytes of quants + one f16 scale each
    last_weight = weight_loads[-1]
    assert any(i < weight_loads[0] for i in loads)     # the activation is requested first
    waits = [int(re.search(r"vmcnt\((\d+)\)", l).group(1)) for l in ins[last_weight:barrier] if "vmcnt" in l]
    assert waits and min(waits) == 6, waits            # staging waits for the activation, not for the weights
    after = [int(re.search(r"vmcnt\((\d+)\)", l).group(1)) for l in ins[barrier:] if "vmcnt" in l]
    first_round = after[:after.index(0) + 1]
    assert sorted(set(first_round), reverse=True) == [4, 2, 0], after   # slot k waits for exactly the loads issued after it
