"""The benchmark driver's contract: one JSON line with the agreed keys, short enough for the
driver's 8 KB tail of stdout, and a refusal of more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode != 0 and "one GPU" in (p.stderr + p.stdout)


def _bench_module():
    sys.path.insert(0, ROOT)
    try:
        import bench
    finally:
        sys.path.remove(ROOT)
    return bench


def test_final_line_fits_the_driver_tail():
    """The line of the default run (headline + a compact record of all twelve workloads) is far below
    the limit, and a result that would not fit loses context keys, never the contract's."""
    bench = _bench_module()
    head = {"metric": "m" * 90, "value": 72662.1, "unit": "tokens/s", "n_gpus": 1, "steps": 20, "warmup": 5,
            "ms_per_step": 0.4404, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
            "data": "synthetic", "config": {"workload": "w" * 120, "path": "p" * 160, "active_experts": 8},
            "roofline": {"bound": "hbm", "kernel": "gate_up_grouped_gemm", "achieved": 6759.8, "peak": 8000.0,
                         "unit": "GB/s", "frac": 0.845, "traffic": 1887085286, "traffic_source": "s" * 60,
                         "algorithmic_bytes": 1883242496, "launch_ms": 0.2786},
            "layer": {"bound": "hbm", "achieved": 6401.4, "peak": 8000.0, "unit": "GB/s", "frac": 0.8002},
            "cpu_baseline": {"value": 65.9, "unit": "tokens/s", "cores": 16, "kind": "port", "sample": "x" * 200,
                             "as_written": {"value": 64.0, "unit": "tokens/s", "sample": "y" * 120}},
            "per_op_us": {n: 33.5 for n in ("router_linear", "moe_select", "gate_up_gemm", "swiglu", "down_gemm",
                                            "moe_reduce")},
            "device_ceilings": {"k" * 40 + str(i): 1000 + i for i in range(6)},
            "companion": {w: {"bound": "mfma", "ms": [4.7368, 4.5004], "layer_frac": [0.4871, 0.5131],
                              "kernel_frac": [0.5512, 0.5463]} for w in bench.COMPANION_WORKLOADS}}
    line = bench.final_line(head)
    assert len(line) < 4500 and json.loads(line) == head
    fat = dict(head, companion={w: {"record": "z" * 2000} for w in bench.COMPANION_WORKLOADS})
    d = json.loads(bench.final_line(fat))
    assert len(json.dumps(d)) <= bench.MAX_LINE and d["companion"] is None and d["dropped_for_length"] == ["companion"]
    for key in ("value", "ms_per_step", "roofline", "layer", "cpu_baseline", "config"):
        assert d[key] == head[key]


@pytest.mark.gpu
def test_default_invocation_line_parses_and_is_short(tmp_path):
    """The driver's own command line (default workload, companions, CPU baseline), with the companion
    set cut to two workloads: one line, under 6000 characters, roofline and cpu_baseline at the top."""
    full = tmp_path / "companions.json"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--steps", "20", "--warmup", "5",
                        "--cpu-seconds", "2", "--companion-set", "decode-T1,fine-T32", "--companion-file", str(full)],
                       capture_output=True, text=True, timeout=280)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [ln for ln in p.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1 and len(lines[0]) < 6000
    assert p.stdout[-8000:].lstrip().startswith("{")        # what a tail of 8000 characters holds is the whole line
    d = json.loads(lines[0])
    assert "dropped_for_length" not in d
    for key in ("value", "ms_per_step", "roofline", "layer", "cpu_baseline", "config", "companion"):
        assert d[key] is not None, key
    assert d["roofline"]["bound"] == "hbm" and d["cpu_baseline"]["kind"] == "port"
    assert set(d["companion"]) == {"decode-T1", "fine-T32"}
    for c in d["companion"].values():
        assert c["bound"] == "hbm" and all(v is not None and v > 0 for v in c["ms"] + c["layer_frac"] + c["kernel_frac"])
    rec = json.loads(full.read_text())
    assert set(rec) == {"decode-T1", "decode-T1, fused forms", "fine-T32", "fine-T32, fused forms"}
    assert all("per_op_us" in r and "roofline" in r for r in rec.values())


@pytest.mark.gpu
def test_bench_json_line():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "decode-T8", "--steps", "5",
                        "--warmup", "2", "--cpu-seconds", "1"], capture_output=True, text=True, timeout=280)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [ln for ln in p.stdout.splitlines() if ln.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["unit"] == "tokens/s"
    assert d["vs_baseline"] is None and d["dtype"] == "f16" and "workload" in d["config"]
    r = d["roofline"]
    assert r["bound"] in ("hbm", "mfma") and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert abs(d["value"] - 8 / (d["ms_per_step"] * 1e-3)) / d["value"] < 1e-3
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["value"] > 0 and "sample" in c
    # what the device sustains, from the probe beside the library: operands that stay in L2 reach LDS
    # faster than operands streamed in the tile kernels' pattern, and both are real rates
    dc = d["device_ceilings"]
    assert dc["hbm_read_nontemporal_GBs"] > 1000 and dc["mfma_f16_16x16x32_lds_fed_TFLOPs"] > 100
    assert dc["tile_operands_to_lds_L2_resident_GBs_per_CU"] > dc["tile_operands_to_lds_streamed_8x4_per_XCD_GBs_per_CU"] > 5
