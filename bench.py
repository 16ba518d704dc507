#!/usr/bin/env python3
"""Benchmark of the MoE layer hot path on one MI355X.

A "step" is one forward pass of the Mixtral-style MoE layer (router gate ->
MoeSelect -> gate/up grouped GEMM -> SwiGLU -> down grouped GEMM -> MoeReduce)
through the drop-in operators, over one batch of synthetic tokens that is
already resident in HBM.  Prints ONE JSON line:

  value / ms_per_step  whole-layer tokens/s and latency over exactly --steps steps (the first timed
                       window, after --warmup untimed steps)
  conditioning         untimed layer steps run before the warm-up (--conditioning-ms of them): a
                       device that has been idle takes some ten milliseconds of work to reach its
                       sustained clocks, more than a short --warmup covers
  windows              ms/step of further windows of --steps steps each (min / median / max)
  roofline             the dominant kernel (gate/up grouped GEMM): algorithmic bytes
                       or flops per launch / mean launch duration (HIP events on
                       the launch stream, taken inside the timed steps) vs MI355X peak
  layer                the same accounting for the whole layer
  hip_graph_replay     the same steps replayed from one captured HIP graph (launch cost of the
                       six operators taken off the host)
  per_op_us            mean duration of each operator (separate untimed pass)
  device_ceilings      streaming-read GB/s, MFMA TFLOP/s (random fp16 operands) and the GB/s
                       per CU at which tile operands reach LDS that this device sustains,
                       from the probe ppl.pmx_amd/lib/opmx_device_ceilings
  vendor_dense_gemm_same_flops_TFLOPs
                       MFMA-bound workloads: the vendor library's dense GEMM with the flop
                       count of the gate/up launch (no expert grouping), context only
  companion            with the default workload: every configuration of the benchmark set
                       (fp32 T=64, decode T=1/8/32/128, T=512/1024, prefill T=2048/8192, 64 experts
                       T=32/4096, 8x22B shape T=16/4096), each as the operator-by-operator sequence and
                       with the fused forms (--fused), measured by child processes of this program: per
                       workload ms per step, whole-layer and dominant-kernel fraction of peak, as
                       [six operators, fused forms]; the children's full records go to stderr and to
                       --companion-file
  cpu_baseline         the CPU oracle (PyTorch CPU restatement of the reference
                       operator sequence) on the host cores, bounded sample

Inputs: x ~ N(0,1) and the router weight ~ N(0,0.02) are drawn on the CPU under
torch.manual_seed(0), x first, so the routing (expert shares, active experts) is that of the seeded
tensor set; the expert weights ~ N(0,0.02), whose values influence neither routing nor timing, are
drawn on the device unless --cpu-weights asks for the CPU draws as well (about a minute).

Workloads (--workload): decode-T{1,8,32,128} and prefill-T{2048,8192} at the
Mixtral-8x7B shape (fp16), fine-T{32,4096} (64 experts, top-8, bf16),
8x22b-T{16,4096}; tiny-T64 (the fp32 configuration: hidden 1024, 8 experts, ffn 2816);
e128-T<n> / e256-T<n>: 128 / 256 small experts (bf16).  Any T is accepted.
Default: decode-T32, the configuration the metric is quoted on.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "ppl.pmx_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, vendor figure
MFMA_PEAK_TFLOPS = 2500.0      # dense fp16/bf16 MFMA, vendor figure
MFMA_PEAK_TFLOPS_F32 = 157.3   # dense fp32 MFMA, vendor figure

# HBM bytes per launch of the dominant kernel come from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs
# of this program, each scaled by the same counter's reading for a plain copy kernel of known size.
# The summaries under profiles/ record them in a line
#   bench-traffic: workload=<name> forms=<none|swiglu|all> bytes_per_launch=<n> kernel_sources_sha256=<hex>
# (forms: which fused forms the run used: none, the SwiGLU epilogue alone, or all three as with --fused)
# together with the hash of the kernel sources the counter run was made with; a line whose hash
# is not that of the sources in this tree is out of date and is not reported.
def kernel_sources_sha256():
    import glob
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "ppl.pmx_amd", "csrc")
    for path in sorted(glob.glob(os.path.join(csrc, "*.hip")) + glob.glob(os.path.join(csrc, "*.h"))):
        if os.path.basename(path) == "device_ceilings.hip":
            continue
        h.update(os.path.basename(path).encode())
        h.update(open(path, "rb").read())
    return h.hexdigest()


def measured_traffic(workload, forms):
    """(bytes per launch or None, where the figure comes from / why there is none)."""
    import glob
    import re
    want = kernel_sources_sha256()
    stale = None
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "*.txt"))):
        for m in re.finditer(r"bench-traffic: workload=(\S+) forms=(\w+) bytes_per_launch=(\d+) "
                             r"kernel_sources_sha256=([0-9a-f]+)", open(path).read()):
            if m.group(1) != workload or m.group(2) != forms:
                continue
            rel = os.path.relpath(path, ROOT)
            if m.group(4) == want:
                return int(m.group(3)), rel
            stale = "{}: counter run made with other kernel sources, not reported".format(rel)
    return None, stale or "no counter run for this workload under profiles/"


# configurations of the benchmark set measured beside the default workload (child processes), each as
# the operator-by-operator sequence and with the fused forms MoeFeedForward uses by default
COMPANION_WORKLOADS = ["tiny-T64", "decode-T1", "decode-T8", "decode-T32", "decode-T128", "decode-T512", "decode-T1024",
                       "prefill-T2048", "prefill-T8192", "fine-T32", "fine-T4096", "8x22b-T16", "8x22b-T4096"]


SHAPES = {
    "decode": dict(H=4096, E=8, k=2, I=14336, dtype="float16", skew=0.0, name="mixtral-8x7b"),
    "prefill": dict(H=4096, E=8, k=2, I=14336, dtype="float16", skew=1.5, name="mixtral-8x7b"),
    "fine": dict(H=2048, E=64, k=8, I=1408, dtype="bfloat16", skew=0.0, name="fine-grained-64x8"),
    "8x22b": dict(H=6144, E=8, k=2, I=16384, dtype="float16", skew=0.0, name="mixtral-8x22b-shape"),
    # the reference's CPU-runnable configuration (fp32): parity case first, here also a measured one
    "tiny": dict(H=1024, E=8, k=2, I=2816, dtype="float32", skew=0.0, name="tiny-fp32"),
    "decodebf": dict(H=4096, E=8, k=2, I=14336, dtype="bfloat16", skew=0.0, name="mixtral-8x7b-bf16"),
    "prefillbf": dict(H=4096, E=8, k=2, I=14336, dtype="bfloat16", skew=1.5, name="mixtral-8x7b-bf16"),
    # further shapes (not part of the reference's configurations): many small experts
    "e128": dict(H=2048, E=128, k=8, I=768, dtype="bfloat16", skew=0.0, name="128-experts-top8-ffn768"),
    "e256": dict(H=7168, E=256, k=8, I=2048, dtype="bfloat16", skew=0.0, name="256-experts-top8-ffn2048"),
}


def parse_workload(w):
    kind, t = w.split("-T")
    cfg = dict(SHAPES[kind])
    cfg["T"] = int(t)
    cfg["kind"] = kind
    return cfg


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="decode-T32")
    ap.add_argument("--conditioning-ms", type=float, default=300.0,
                    help="untimed layer steps for this long before the warm-up (reported, never timed)")
    ap.add_argument("--windows", type=int, default=4, help="further timed windows of --steps steps (min/median/max)")
    ap.add_argument("--cpu-weights", action="store_true",
                    help="draw the expert weights on the CPU too, after x and the router weight (slow)")
    ap.add_argument("--no-graph", action="store_true", help="skip the HIP-graph replay leg")
    ap.add_argument("--event-stride", type=int, default=8,
                    help="HIP events around every n-th launch of the dominant kernel inside the timed steps")
    ap.add_argument("--fuse-router-select", action="store_true",
                    help="router gate and MoeSelect through the fused call (one launch up to 8 tokens)")
    ap.add_argument("--fuse-swiglu", action="store_true", help="apply SwiGLU in the gate/up GEMM epilogue")
    ap.add_argument("--fuse-gather", action="store_true",
                    help="MoeSelect returns an index instead of the expanded copy of the tokens; the gate/up GEMM "
                         "reads its rows through it")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the CPU baseline leg")
    ap.add_argument("--no-device-ceilings", action="store_true",
                    help="skip the probe of the HBM-read / MFMA rates this device sustains")
    ap.add_argument("--no-vendor-gemm", action="store_true",
                    help="MFMA-bound workloads: skip timing the vendor dense GEMM of the same flop count")
    ap.add_argument("--no-companion", action="store_true",
                    help="with the default workload, do not also measure the MFMA-bound prefill workload")
    ap.add_argument("--companion-set", default="", metavar="W1,W2",
                    help="measure only these workloads beside the default one (default: the whole benchmark set)")
    ap.add_argument("--companion-file", default=os.path.join(ROOT, "gpurun_out", "bench_companions.json"),
                    help="where the companion workloads' full records are written (the final line holds three "
                         "figures per workload)")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="N",
                    help="also run N plain device-to-device copies of the gate/up weight tensor (known size): "
                         "the reference reading for FETCH_SIZE / WRITE_SIZE counter runs")
    ap.add_argument("--kernel-sources-hash", action="store_true",
                    help="print the hash that a bench-traffic line under profiles/ must carry for this tree, and exit")
    ap.add_argument("--fused", action="store_true",
                    help="all three fused forms (--fuse-swiglu --fuse-gather --fuse-router-select): the block as "
                         "MoeFeedForward runs it by default")
    args = ap.parse_args()
    if args.fused:
        args.fuse_swiglu = args.fuse_gather = args.fuse_router_select = True
    if args.kernel_sources_hash:
        print(kernel_sources_sha256())
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (TP=1, no collectives); --gpus {} is not "
                 "supported, run with --gpus 1".format(args.gpus))

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X (no GPU visible)")

    # What this device sustains (streaming read, MFMA on random operands): a child process,
    # run before this process touches the GPU.  Context for the roofline fractions only.
    ceilings = None
    probe = os.path.join(ROOT, "ppl.pmx_amd", "lib", "opmx_device_ceilings")
    if not args.no_device_ceilings and os.path.exists(probe):
        import subprocess
        try:
            ceilings = json.loads(subprocess.run([probe], capture_output=True, text=True, timeout=120,
                                                 check=True).stdout.strip().splitlines()[-1])
        except Exception as exc:   # the probe is optional
            print("device ceiling probe failed: {}".format(exc), file=sys.stderr)
    # The default run also measures every other configuration of the benchmark set: child
    # processes of this program, run one after the other while this one leaves the GPU idle.
    # The final JSON line carries three figures per configuration (ms per step, whole-layer
    # fraction of peak, dominant-kernel fraction of peak; [six operators, fused forms]); the
    # children's full records go to stderr, one line each, and to --companion-file.
    companion = None
    if args.workload == "decode-T32" and not args.no_companion:
        import subprocess
        names = [w.strip() for w in args.companion_set.split(",") if w.strip()] if args.companion_set else COMPANION_WORKLOADS
        companion, full = {}, {}
        for name in names:
            entry = {"bound": None, "ms": [None, None], "layer_frac": [None, None], "kernel_frac": [None, None]}
            for slot, extra in enumerate(([], ["--fused"])):
                if name == "decode-T32" and not extra:
                    continue            # the headline itself, filled in below
                cmd = [sys.executable, os.path.abspath(__file__), "--workload", name, "--steps", "40", "--warmup", "5",
                       "--windows", "2", "--conditioning-ms", "200", "--no-cpu-baseline", "--no-device-ceilings",
                       "--no-vendor-gemm", "--no-companion"] + extra
                try:
                    line = subprocess.run(cmd, capture_output=True, text=True, timeout=300, check=True).stdout.strip().splitlines()[-1]
                    r = json.loads(line)
                    full[name + (", fused forms" if extra else "")] = r
                    print("companion {}{}: {}".format(name, " --fused" if extra else "", line), file=sys.stderr)
                    entry["bound"] = r["layer"]["bound"]
                    entry["ms"][slot] = r["ms_per_step"]
                    entry["layer_frac"][slot] = r["layer"]["frac"]
                    entry["kernel_frac"][slot] = r["roofline"]["frac"]
                except Exception as exc:
                    print("companion workload {} failed: {}".format(name, exc), file=sys.stderr)
            companion[name] = entry
        try:
            os.makedirs(os.path.dirname(os.path.abspath(args.companion_file)), exist_ok=True)
            with open(args.companion_file, "w") as f:
                json.dump(full, f, indent=1)
        except OSError as exc:
            print("companion records not written to {}: {}".format(args.companion_file, exc), file=sys.stderr)

    import torch_function as OPMX
    from model_zoo.mixtral.modeling.dynamic_batching.Model import MoeFeedForward

    cfg = parse_workload(args.workload)
    T, H, E, k, I = cfg["T"], cfg["H"], cfg["E"], cfg["k"], cfg["I"]
    dtype = getattr(torch, cfg["dtype"])
    s = 4 if cfg["dtype"] == "float32" else 2
    mfma_peak = MFMA_PEAK_TFLOPS_F32 if cfg["dtype"] == "float32" else MFMA_PEAK_TFLOPS
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    # ---- synthetic inputs: x and the router weight from the CPU generator under seed 0 (x first),
    # so the routing is that of the seeded tensor set; expert weights on the device (see above)
    gc = torch.Generator().manual_seed(0)
    x = torch.randn(T, H, generator=gc).to(dtype).to(dev)
    layer = MoeFeedForward(MoeFeedForward.params(H, I, E, k), 0, True, False, None, dtype=dtype, device=dev,
                           fuse_swiglu_epilogue=args.fuse_swiglu)
    layer.gate.weight.data = (torch.randn(E, H, generator=gc) * 0.02).to(dtype).to(dev)
    g = torch.Generator(device="cuda").manual_seed(0)
    if args.cpu_weights:
        for e in range(E):
            layer.wu.weight.data[e] = (torch.randn(2 * I, H, generator=gc) * 0.02).to(dtype).to(dev)
        for e in range(E):
            layer.w2.weight.data[e] = (torch.randn(H, I, generator=gc) * 0.02).to(dtype).to(dev)
    else:
        for e in range(E):
            layer.wu.weight.data[e] = (torch.randn(2 * I, H, generator=g, device=dev) * 0.02).to(dtype)
            layer.w2.weight.data[e] = (torch.randn(H, I, generator=g, device=dev) * 0.02).to(dtype)
    if cfg["skew"] > 0:       # Zipf(s=1.2) per-expert logit bias: skewed expert load
        p = torch.arange(1, E + 1, dtype=torch.float64) ** -1.2
        bias = (cfg["skew"] * torch.log(p / p.sum())).to(dtype).to(dev)
        layer.gate.bias = torch.nn.Parameter(bias, requires_grad=False)
    Wg, wu, w2, gb = layer.gate.weight, layer.wu.weight, layer.w2.weight, layer.gate.bias

    # router gate and MoeSelect in the form the flags ask for -> (xe, w, inv, off); with --fuse-gather
    # `xe` is the index that stands for the expanded copy
    def timed_select(timed):
        if args.fuse_gather:
            if args.fuse_router_select:
                w, inv, off, rt, sc = timed("router_and_select", lambda: OPMX.moe_route_select_index(x, Wg, gb, E, k))
            else:
                sc = timed("router_linear", lambda: OPMX.linear(x, Wg, gb, H, E))
                w, inv, off, rt = timed("moe_select", lambda: OPMX.moe_select_index(sc, E, k))
            return rt, w, inv, off
        if args.fuse_router_select:
            xe, w, inv, off, sc = timed("router_and_select", lambda: OPMX.moe_route_select(x, Wg, gb, E, k))
        else:
            sc = timed("router_linear", lambda: OPMX.linear(x, Wg, gb, H, E))
            xe, w, inv, off = timed("moe_select", lambda: OPMX.moe_select(x, sc, E, k))
        return xe, w, inv, off

    def gemm1(xe, off):
        if args.fuse_gather:
            return OPMX.moe_column_parallel_linear_indexed(x, xe, off, wu, None, E, H, 2 * I, swiglu=args.fuse_swiglu)
        if args.fuse_swiglu:
            return OPMX.moe_column_parallel_linear_swiglu(xe, off, wu, None, E, H, 2 * I)
        return OPMX.moe_column_parallel_linear(xe, off, wu, None, None, E, H, 2 * I, False)

    # ---- one instrumented pass: routing statistics + per-operator durations
    def ops(record=None):
        def timed(name, fn):
            if record is None:
                return fn()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            r = fn()
            b.record()
            record.append((name, a, b))
            return r
        xe, w, inv, off = timed_select(timed)
        if args.fuse_swiglu:
            act = timed("gate_up_gemm", lambda: gemm1(xe, off))
        else:
            h = timed("gate_up_gemm", lambda: gemm1(xe, off))
            act = timed("swiglu", lambda: OPMX.swiglu(h))
        y = timed("down_gemm", lambda: OPMX.moe_row_parallel_linear(act, off, w2, None, None, E, I, H, True))
        out = timed("moe_reduce", lambda: OPMX.moe_reduce(y, w, inv, k))
        return out, off

    def step(i=-1, ev=None, stride=1):
        xe, w, inv, off = timed_select(lambda name, fn: fn())
        mark = ev is not None and i % stride == 0
        if mark:
            ev[i // stride][0].record()
        h = gemm1(xe, off)
        if mark:
            ev[i // stride][1].record()
        act = h if args.fuse_swiglu else OPMX.swiglu(h)
        y = OPMX.moe_row_parallel_linear(act, off, w2, None, None, E, I, H, True)
        return OPMX.moe_reduce(y, w, inv, k)

    def window(n, ev=None, stride=1):
        """n steps between two device synchronisations -> ms per step"""
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            step(i, ev, stride)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e3

    with torch.inference_mode():
        out, off = ops()
        torch.cuda.synchronize()
        counts = (off[1:] - off[:-1]).cpu()
        active = int((counts > 0).sum())
        R = T * k
        if cfg["kind"] == "prefill":
            assert float(counts.max()) / R > 0.40, "skewed-routing config needs the largest expert above 40%"

        # ---- conditioning (untimed, reported): layer steps until the device has been busy for
        # --conditioning-ms.  Straight out of idle the same kernels run 8-10 % slower for the first
        # ten milliseconds or so, which a warm-up of a few steps does not cover.
        cond_steps, c0 = 0, time.perf_counter()
        while (time.perf_counter() - c0) * 1e3 < args.conditioning_ms:
            for _ in range(8):
                step()
            cond_steps += 8
            torch.cuda.synchronize()
        cond_ms = (time.perf_counter() - c0) * 1e3

        # ---- warm-up, then the timed region: exactly --steps steps; HIP events bracket the dominant
        # kernel at every `stride`-th launch (at least 8 of them): an event record is a barrier
        # packet in the queue, and two per step cost the eager steps 1-3 %
        for _ in range(args.warmup):
            step()
        stride = max(1, min(args.event_stride, args.steps // 8 if args.steps >= 8 else 1))
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
              for _ in range((args.steps + stride - 1) // stride)]
        ms_per_step = window(args.steps, ev, stride)
        gemm1_ms = sum(a.elapsed_time(b) for a, b in ev) / len(ev)
        # further windows of the same length, for the spread
        more = sorted(window(args.steps) for _ in range(max(args.windows, 0)))
        windows = None
        if more:
            windows = {"n": len(more), "steps_each": args.steps, "ms_per_step_min": round(more[0], 4),
                       "ms_per_step_median": round(more[len(more) // 2] if len(more) % 2 else
                                                   0.5 * (more[len(more) // 2 - 1] + more[len(more) // 2]), 4),
                       "ms_per_step_max": round(more[-1], 4)}

        # ---- the same steps replayed from a captured HIP graph: what a serving loop does when the
        # host's launch path (six operators per layer) is slower than the GPU work, i.e. at few
        # tokens.  Reported beside `value`, which stays the eager operator sequence.
        graph_ms = None
        if not args.no_graph:
            try:
                torch.cuda.synchronize()
                cg = torch.cuda.CUDAGraph()
                with torch.cuda.graph(cg):
                    ops()
                c0 = time.perf_counter()
                while (time.perf_counter() - c0) * 1e3 < args.conditioning_ms / 3:
                    for _ in range(8):
                        cg.replay()
                    torch.cuda.synchronize()
                for _ in range(args.warmup):
                    cg.replay()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(args.steps):
                    cg.replay()
                torch.cuda.synchronize()
                graph_ms = (time.perf_counter() - t0) / args.steps * 1e3
                del cg
            except Exception as exc:
                print("graph replay leg failed: {}".format(exc), file=sys.stderr)

        # ---- per-operator durations (untimed extra pass, averaged)
        per_op = {}
        reps = 20
        for _ in range(reps):
            rec = []
            ops(rec)
            torch.cuda.synchronize()
            for name, a, b in rec:
                per_op[name] = per_op.get(name, 0.0) + a.elapsed_time(b) * 1e3 / reps

    # Context for MFMA-bound workloads: the vendor library's dense GEMM (hipBLASLt behind
    # torch.nn.functional.linear) on [R, H] x [2I, H]^T, the flop count of the gate/up launch
    # without expert grouping or ragged tiles, same random operands, measured the same way.
    vendor_tflops = None
    if cfg["kind"] != "decode" and T >= 1024 and not args.no_vendor_gemm:
        with torch.inference_mode():
            xe_d = torch.randn(T * k, H, generator=g, device=dev).to(dtype)
            for _ in range(3):
                torch.nn.functional.linear(xe_d, wu[0])
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(10):
                torch.nn.functional.linear(xe_d, wu[0])
            b.record()
            torch.cuda.synchronize()
            vendor_tflops = round(2.0 * T * k * H * 2 * I / (a.elapsed_time(b) / 10 * 1e-3) / 1e12, 1)
            del xe_d

    if args.copy_calibration > 0:
        dst = torch.empty_like(wu)
        for _ in range(args.copy_calibration):
            dst.copy_(wu)
        torch.cuda.synchronize()
        print("copy calibration: {} copies of {} bytes (read) + {} bytes (written)".format(
            args.copy_calibration, wu.numel() * s, wu.numel() * s), file=sys.stderr)

    # ---- algorithmic work
    w_bytes_gemm1 = active * 2 * I * H * s
    w_bytes_gemm2 = active * H * I * s
    n1 = I if args.fuse_swiglu else 2 * I
    gemm1_bytes = w_bytes_gemm1 + R * H * s + R * n1 * s
    gemm1_flops = 2.0 * R * H * 2 * I
    layer_bytes = w_bytes_gemm1 + w_bytes_gemm2 + 2 * T * H * s + E * H * s
    layer_flops = T * (k * (2.0 * H * 2 * I + 2.0 * I * H) + 2.0 * H * E)
    fl = (args.fuse_swiglu, args.fuse_gather, args.fuse_router_select)
    forms = {(False, False, False): "none", (True, False, False): "swiglu", (True, True, True): "all"}.get(fl, "other")
    traffic, traffic_source = measured_traffic(args.workload, forms)
    hbm_bound = (layer_flops / layer_bytes) < (mfma_peak * 1e12) / (HBM_PEAK_GBS * 1e9)
    if hbm_bound:
        ach = gemm1_bytes / (gemm1_ms * 1e-3) / 1e9
        roof = dict(bound="hbm", kernel="gate_up_grouped_gemm", achieved=round(ach, 1), peak=HBM_PEAK_GBS,
                    unit="GB/s", frac=round(ach / HBM_PEAK_GBS, 4),
                    traffic=traffic, traffic_source=traffic_source,
                    algorithmic_bytes=int(gemm1_bytes), launch_ms=round(gemm1_ms, 4))
        lach = layer_bytes / (ms_per_step * 1e-3) / 1e9
        lay = dict(bound="hbm", achieved=round(lach, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                   frac=round(lach / HBM_PEAK_GBS, 4), algorithmic_bytes=int(layer_bytes))
    else:
        ach = gemm1_flops / (gemm1_ms * 1e-3) / 1e12
        roof = dict(bound="mfma", kernel="gate_up_grouped_gemm", achieved=round(ach, 1), peak=mfma_peak,
                    unit="TFLOP/s", frac=round(ach / mfma_peak, 4),
                    traffic=traffic, traffic_source=traffic_source,
                    algorithmic_flops=int(gemm1_flops), launch_ms=round(gemm1_ms, 4))
        lach = layer_flops / (ms_per_step * 1e-3) / 1e12
        lay = dict(bound="mfma", achieved=round(lach, 1), peak=mfma_peak, unit="TFLOP/s",
                   frac=round(lach / mfma_peak, 4), algorithmic_flops=int(layer_flops))

    if ceilings:
        if hbm_bound:
            roof["measured_ceiling"] = ceilings["hbm_read_nontemporal_GBs"]
        else:
            roof["measured_ceiling"] = ceilings.get("mfma_f16_16x16x32_lds_fed_TFLOPs", ceilings["mfma_f16_lds_fed_TFLOPs"])
        roof["frac_of_measured_ceiling"] = round(roof["achieved"] / roof["measured_ceiling"], 4)

    result = {
        "metric": "MoE-layer tokens/sec at Mixtral-8x7B shape, fp16, 1 GPU; % HBM/MFMA roofline",
        "value": round(T / (ms_per_step * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "conditioning": {"steps": cond_steps, "ms": round(cond_ms, 1), "timed": False}, "windows": windows,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"float16": "f16", "bfloat16": "bf16", "float32": "f32"}[cfg["dtype"]], "data": "synthetic",
        "config": {"workload": "{} MoE layer {}, T={} tokens, hidden={}, experts={}, top-{}, ffn={}, TP=1".format(
            cfg["name"], "decode" if hbm_bound else "prefill", T, H, E, k, I),
            "path": "drop-in operator sequence" + (" + fused SwiGLU epilogue" if args.fuse_swiglu else "")
            + (" + router gate and select in one call" if args.fuse_router_select else "")
            + (" + token gather folded into the gate/up GEMM" if args.fuse_gather else ""),
            "active_experts": active, "max_expert_share": round(float(counts.max()) / R, 3)},
        "roofline": roof, "layer": lay,
        "hip_graph_replay": None if graph_ms is None else {"ms_per_step": round(graph_ms, 4),
                                                           "value": round(T / (graph_ms * 1e-3), 1), "unit": "tokens/s"},
        "per_op_us": {n: round(v, 1) for n, v in per_op.items()},
        "device_ceilings": ceilings, "companion": companion, "vendor_dense_gemm_same_flops_TFLOPs": vendor_tflops, "device": torch.cuda.get_device_name(0), "cu_count": torch.cuda.get_device_properties(0).multi_processor_count,
    }

    # ---- CPU baseline: the oracle (PyTorch CPU restatement of the reference operator
    # sequence) on this box's host cores.  Checker code, timed only here.
    if not args.no_cpu_baseline:
        from oracle import moe_oracle as O
        Tc = T if T <= 512 else 512            # bounded sample of the same workload
        xc, Wgc, wuc, w2c = x[:Tc].cpu(), Wg.cpu(), wu.cpu(), w2.cpu()
        gbc = None if gb is None else gb.cpu()
        def timed_runs(budget, **kw):
            runs, spent = 0, 0.0
            while runs < 1 or (spent < budget and runs < 20):
                c0 = time.perf_counter()
                O.moe_layer(xc, Wgc, wuc, w2c, E, k, router_bias=gbc, round_between_ops=True, **kw)
                spent += time.perf_counter() - c0
                runs += 1
            return runs, spent
        runs, spent = timed_runs(args.cpu_seconds * 0.7)
        runs_w, spent_w = timed_runs(args.cpu_seconds * 0.3, as_written=True)
        result["cpu_baseline"] = {
            "value": round(Tc / (spent / runs), 2), "unit": "tokens/s", "cores": torch.get_num_threads(),
            "kind": "port", "host_cpus": os.cpu_count(),
            "sample": "{} run(s) of the same layer on the first {} tokens, fp32 accumulation on {} inputs, "
                      "{:.1f} s of CPU time (vectorised routing bookkeeping)".format(runs, Tc, cfg["dtype"], spent),
            "as_written": {"value": round(Tc / (spent_w / runs_w), 2), "unit": "tokens/s",
                           "sample": "{} run(s), routing bookkeeping in interpreted per-element loops as in the "
                                     "reference, {:.1f} s".format(runs_w, spent_w)}}
    if companion and "decode-T32" in companion:     # the headline is the six-operator form of this workload
        c = companion["decode-T32"]
        c["bound"], c["ms"][0], c["layer_frac"][0], c["kernel_frac"][0] = lay["bound"], result["ms_per_step"], lay["frac"], roof["frac"]
    if companion:
        result["companion_legend"] = ("per workload: ms per step, whole-layer and dominant-kernel fraction of the "
                                      "peak named by bound; each as [six operators, fused forms]; full records: "
                                      + os.path.relpath(args.companion_file, ROOT))
    print(final_line(result))


# The benchmark driver keeps the last 8 KB of stdout: the one JSON line must fit with room to spare.
MAX_LINE = 6000
OPTIONAL_KEYS = ("device_ceilings", "per_op_us", "companion_legend", "conditioning", "windows", "hip_graph_replay",
                 "companion")


def final_line(result):
    """The JSON line of a result; while it is longer than MAX_LINE characters the largest of the
    context-only keys is dropped (the keys the contract names are never dropped)."""
    result = dict(result)
    line = json.dumps(result)
    dropped = []
    while len(line) > MAX_LINE:
        sizes = sorted((len(json.dumps(result[key])), key) for key in OPTIONAL_KEYS if result.get(key) is not None)
        if not sizes:
            break
        result[sizes[-1][1]] = None
        dropped.append(sizes[-1][1])
        result["dropped_for_length"] = dropped
        line = json.dumps(result)
    return line


if __name__ == "__main__":
    main()
