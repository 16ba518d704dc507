#!/usr/bin/env python3
"""Static checks on the gfx950 assembly of the direct-to-LDS grouped GEMM kernel.

The kernel (gemm_tiled_dlds_kernel in moe_gemm_tiled.hip) issues its MFMAs from inline assembly
and counts its own outstanding loads, so three things the compiler normally guarantees have to be
checked on its output instead:

1. no instruction other than an MFMA touches an accumulator register between the first MFMA and
   the wait that lets the last MFMAs retire (the compiler adds no hazard padding behind inline
   assembly: a copy or spill placed right behind an MFMA would read the old value);
2. no buffer load sits in a loop over lanes (a descriptor the compiler cannot prove uniform), and
   nothing spills to scratch memory inside the k loop: both would add memory operations the
   hand-written `s_waitcnt vmcnt(N)` counts know nothing about;
3. the k loop holds exactly the MFMAs, LDS reads and loads of one k-tile.

usage: check_kernel_asm.py file.s   (hipcc -S --cuda-device-only output); exit status 1 on a finding
"""
import re
import sys

KERNEL = re.compile(r"^(_Z\S*gemm_tiled_dlds_kernel\S*):")
AGPR = re.compile(r"\ba(\[\d+:\d+\]|\d+\b)")


def functions(lines):
    name, body = None, []
    for ln in lines:
        m = KERNEL.match(ln)
        if m:
            name, body = m.group(1), []
        elif name is not None:
            if ln.startswith(".Lfunc_end"):
                yield name, body
                name = None
            else:
                body.append(ln)


def check(path):
    findings, seen = [], 0
    for name, body in functions(open(path).read().split("\n")):
        seen += 1
        code = [(i, l.strip()) for i, l in enumerate(body) if l.strip() and not l.strip().startswith(";")]
        text = [l for _, l in code]
        mfma = [k for k, l in enumerate(text) if l.startswith("v_mfma")]
        nops = [k for k, l in enumerate(text) if l.startswith("s_nop 15")]
        if not mfma or not nops:
            findings.append((name, "no MFMA / no retire wait found"))
            continue
        # 1. accumulators between first MFMA and the retire wait (zero-initialisation excluded)
        for l in text[mfma[0]:nops[-1]]:
            if AGPR.search(l) and not l.startswith(("v_mfma", "v_accvgpr_write", "v_accvgpr_mov")):
                findings.append((name, "accumulator touched before the MFMAs retired: " + l))
        # 2a. loads into LDS under a per-lane loop: preceded by s_and_saveexec
        for k, l in enumerate(text):
            if l.startswith("buffer_load") and " lds" in l and k and text[k - 1].startswith("s_and_saveexec"):
                findings.append((name, "direct-to-LDS load inside a loop over lanes"))
                break
        # 2b/3. the k loop: the innermost loop holding the most MFMAs
        loops, start = [], None
        for k, l in enumerate(text):
            if re.match(r"^\.LBB\d+_\d+:", l):
                start = (k, l.split(":")[0])
            m = re.match(r"^s_cbranch_\w+ (\.LBB\d+_\d+)", l)
            if m and start and m.group(1) == start[1]:
                loops.append(text[start[0]:k + 1])
        kloop = max(loops, key=lambda b: sum(x.startswith("v_mfma") for x in b), default=[])
        count = lambda p: sum(x.startswith(p) for x in kloop)
        if (count("v_mfma"), count("ds_read_b128"), count("buffer_load_dwordx4")) != (128, 32, 16):
            findings.append((name, "k loop holds {} MFMAs, {} LDS reads, {} loads (expected 128, 32, 16)".format(
                count("v_mfma"), count("ds_read_b128"), count("buffer_load_dwordx4"))))
        if any(x.startswith("scratch_") for x in kloop):
            findings.append((name, "scratch access inside the k loop"))
    if seen == 0:
        findings.append(("-", "no gemm_tiled_dlds_kernel in " + path))
    return seen, findings


if __name__ == "__main__":
    n, found = check(sys.argv[1])
    for name, what in found:
        print("{}: {}".format(name, what))
    print("{} kernels checked, {} findings".format(n, len(found)))
    sys.exit(1 if found else 0)
