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
3. the k loop (the loop with the most MFMAs, by the compiler's loop annotations) holds exactly
   the MFMAs, LDS reads and loads of one k-tile;
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


def blocks(body):
    """Splits a function body into basic blocks using the compiler's own annotations: returns
    (instructions, per-instruction innermost loop header or None, parent header of each header,
    headers of loops without inner loops)."""
    text, where, parent, innermost = [], [], {}, set()
    cur = None            # innermost loop header of the current block
    pending_label = None
    for raw in body:
        line = raw.strip()
        m = re.match(r"^(?:\.LBB\d+_(\d+):|; %bb\.(\d+):)\s*(;.*)?$", line)
        if m:
            pending_label = m.group(1) or m.group(2)
            cur = None
            line = m.group(3) or ""
        if line.startswith(";"):
            if pending_label is not None:
                h = re.search(r"in Loop: Header=BB\d+_(\d+) Depth=\d+", line)
                if h:
                    cur = h.group(1)
                if re.search(r"This (Inner )?Loop Header: Depth=\d+", line):
                    cur = pending_label
                    if "Inner" in line:
                        innermost.add(pending_label)
                pl = re.findall(r"Parent Loop BB\d+_(\d+) Depth=\d+", line)
                if pl:
                    parent.setdefault(pending_label, []).extend(pl)
            continue
        if not line:
            continue
        text.append(line)
        where.append(cur)
    # the innermost parent is the last "Parent Loop" line of a header
    return text, where, {h: ps[-1] for h, ps in parent.items()}, innermost


def check(path):
    findings, seen = [], 0
    for name, body in functions(open(path).read().split("\n")):
        seen += 1
        text, where, parent, innermost = blocks(body)
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
        # 2b/3. the k loop: the innermost loop with the most MFMAs
        per_loop = {}
        for l, h in zip(text, where):
            if h is not None:
                per_loop.setdefault(h, []).append(l)
        khead = max((h for h in per_loop if h in innermost),
                    key=lambda h: sum(x.startswith("v_mfma") for x in per_loop[h]), default=None)
        kloop = per_loop.get(khead, [])
        count = lambda p: sum(x.startswith(p) for x in kloop)
        # 256 x 256 tiles (template arguments <T, 256, 256, ...>) or 128 x 256
        expected = (64, 24, 12) if "Li128ELi256E" in name else (128, 32, 16)
        if (count("v_mfma"), count("ds_read_b128"), count("buffer_load_dwordx4")) != expected:
            findings.append((name, "k loop holds {} MFMAs, {} LDS reads, {} loads (expected {}, {}, {})".format(
                count("v_mfma"), count("ds_read_b128"), count("buffer_load_dwordx4"), *expected)))
        if any(x.startswith("scratch_") for x in kloop):
            findings.append((name, "scratch access inside the k loop"))
        # 4. persistent kernel: the wait counts assume a fixed number of output stores per wave and
        #    tile (8, 16 or 32), the same number of priming stores before the tile loop, and no other
        #    store in the loop
        if "persist" in name:
            thead = parent.get(khead)
            if thead is None:
                findings.append((name, "no loop over tiles found"))
            else:
                def inside(h):
                    while h is not None:
                        if h == thead:
                            return True
                        h = parent.get(h)
                    return False
                tile = [l for l, h in zip(text, where) if inside(h)]
                rest = [l for l, h in zip(text, where) if not inside(h)]
                st = lambda part: sum(x.startswith("buffer_store_dwordx4") for x in part)
                if st(rest) not in (8, 16, 32) or st(tile) != st(rest):
                    findings.append((name, "{} priming stores, {} stores in the tile loop".format(st(rest), st(tile))))
                # ... and that nothing in the tile loop drains the loads and stores kept in flight
                # across tiles: no scratch traffic, no wait for all vector-memory operations
                for l in tile:
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
