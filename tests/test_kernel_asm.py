"""CPU check of the compiled direct-to-LDS GEMM kernel: the MFMAs are issued from inline assembly
and the loads are counted by hand, so what the compiler placed around them is verified on the
gfx950 assembly (no accumulator access before the MFMAs retired, no per-lane load loops, no
scratch traffic in the k loop).  hipcc cross-compiles without a GPU."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "ppl.pmx_amd", "csrc")


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_inline_mfma_kernel_assembly_is_hazard_free():
    r = subprocess.run(["make", "-C", CSRC, "check"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    import re
    m = re.search(r"(\d+) kernels checked, (\d+) findings", r.stdout)
    assert m and int(m.group(1)) >= 1 and int(m.group(2)) == 0, r.stdout[-2000:]


def test_checker_flags_a_copy_behind_an_mfma(tmp_path):
    import sys
    sys.path.insert(0, CSRC)
    import check_kernel_asm as C
    good = ["_Z4x22gemm_tiled_dlds_kernelIfE:", ".LBB0_1:            ; =>This Inner Loop Header: Depth=1"] + \
        ["\tv_mfma_f32_16x16x32_f16 a[0:3], v[0:3], v[4:7], a[0:3]"] * 128 + \
        ["\tds_read_b128 v[0:3], v9"] * 32 + ["\tbuffer_load_dwordx4 v1, s[0:3], 0 offen lds"] * 16 + \
        ["\ts_cbranch_scc1 .LBB0_1", "; %bb.2:", "\ts_nop 15", "\tv_accvgpr_read_b32 v1, a0", ".Lfunc_end0:"]
    p = tmp_path / "good.s"
    p.write_text("\n".join(good))
    assert C.check(str(p)) == (1, [])
    bad = list(good)
    bad.insert(10, "\tscratch_store_dwordx4 off, a[0:3], off offset:16")
    p.write_text("\n".join(bad))
    n, found = C.check(str(p))
    assert n == 1 and any("accumulator touched" in w for _, w in found) and any("scratch" in w for _, w in found)
    bad = list(good)
    bad.insert(170, "\ts_and_saveexec_b64 s[0:1], s[0:1]")
    p.write_text("\n".join(bad))
    assert any("loop over lanes" in w for _, w in C.check(str(p))[1])
