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
3. the k loop (the innermost loop with the most MFMAs) holds exactly the MFMAs, LDS reads and
   loads of one k-tile;
4. the persistent kernel issues the number of output stores per tile that its wait counts assume,
   and its tile loop has no scratch access and no wait that would drain the pipeline.

usage: check_kernel_asm.py file.s   (hipcc -S --cuda-device-only output); exit status 1 on a finding
"""
import re
import sys

KERNEL = re.compile(r"^(_Z\S*gemm_tiled_dlds_(?:persist_)?kernel\S*):")
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
        # 1. walking the code in layout order: after an MFMA no other instruction may touch an
        #    accumulator register until the retire wait (s_nop 15) has been passed
        pending = False
        for l in text:
            if l.startswith("v_mfma"):
                pending = True
            elif l.startswith("s_nop 15"):
                pending = False
            elif pending and AGPR.search(l) and not l.startswith(("v_accvgpr_write", "v_accvgpr_mov")):   # zero fill
                findings.append((name, "accumulator touched before the MFMAs retired: " + l))
        # 2a. loads into LDS under a per-lane loop: preceded by s_and_saveexec
        for k, l in enumerate(text):
            if l.startswith("buffer_load") and " lds" in l and k and text[k - 1].startswith("s_and_saveexec"):
                findings.append((name, "direct-to-LDS load inside a loop over lanes"))
                break
        # 2b/3. the k loop: the innermost loop holding the most MFMAs
        labels = {l.split(":")[0]: k for k, l in enumerate(text) if re.match(r"^\.LBB\d+_\d+:", l)}
        spans = []
        for k, l in enumerate(text):
            m = re.match(r"^s_cbranch_\w+ (\.LBB\d+_\d+)", l)
            if m and labels.get(m.group(1), k + 1) <= k:          # a backward branch closes a loop
                spans.append((labels[m.group(1)], k))
        inner = [(a, z) for a, z in spans if not any((a2, z2) != (a, z) and a <= a2 and z2 <= z for a2, z2 in spans)]
        kspan = max(inner, key=lambda t: sum(x.startswith("v_mfma") for x in text[t[0]:t[1] + 1]), default=(0, -1))
        kloop = text[kspan[0]:kspan[1] + 1]
        count = lambda p: sum(x.startswith(p) for x in kloop)
        if (count("v_mfma"), count("ds_read_b128"), count("buffer_load_dwordx4")) != (128, 32, 16):
            findings.append((name, "k loop holds {} MFMAs, {} LDS reads, {} loads (expected 128, 32, 16)".format(
                count("v_mfma"), count("ds_read_b128"), count("buffer_load_dwordx4"))))
        if any(x.startswith("scratch_") for x in kloop):
            findings.append((name, "scratch access inside the k loop"))
        # 4. persistent kernel: the wait counts assume a fixed number of output stores per wave and
        #    tile (16 or 32), the same number of priming stores before the tile loop, and no other
        #    store in the loop
        if "persist" in name:
            outer = [(a, z) for a, z in spans if a <= kspan[0] and kspan[1] <= z and (a, z) != kspan]
            if not outer:
                findings.append((name, "no loop over tiles found"))
            else:
                a, z = min(outer, key=lambda t: t[1] - t[0])
                st = lambda part: sum(x.startswith("buffer_store_dwordx4") for x in part)
                before, inside = st(text[:a]), st(text[a:z + 1])
                if before not in (16, 32) or inside != before or st(text[z + 1:]) != 0:
                    findings.append((name, "{} priming stores, {} stores in the tile loop".format(before, inside)))
                # ... and that nothing in the tile loop drains the loads and stores kept in flight
                # across tiles: no scratch traffic, no wait for all vector-memory operations
                for l in text[a:z + 1]:
                    if l.startswith("scratch_") or re.match(r"s_waitcnt .*vmcnt\(0\)", l):
                        findings.append((name, "in the tile loop: " + l))
    if seen == 0:
        findings.append(("-", "no gemm_tiled_dlds_kernel in " + path))
    return seen, findings


if __name__ == "__main__":
    n, found = check(sys.argv[1])
    for name, what in found:
        print("{}: {}".format(name, what))
    print("{} kernels checked, {} findings".format(n, len(found)))
    sys.exit(1 if found else 0)
