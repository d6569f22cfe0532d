"""The benchmark's command-line contract: one JSON line with the agreed keys, and a refusal of
more than one GPU.  The GPU leg runs the real thing briefly; the refusal needs no GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True, timeout=120)
    assert run.returncode != 0 and "one GPU" in run.stderr and run.stdout.strip() == ""


def test_the_traffic_and_instruction_tables_quote_the_committed_profile_summaries():
    # `roofline.traffic` and `valu_floor_ms` are not measured inside the bench process: they are the
    # counter results of the profile summaries.  A table entry that no summary holds has gone stale.
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    text = {f: open(os.path.join(ROOT, "profiles", f)).read() for f in os.listdir(os.path.join(ROOT, "profiles"))}
    where = {("base", "duo", 4096): "duo_kernel_int8_batch4096.md", ("base", "twin", 4096): "board_kernel_twin_int8_batch4096.md",
             ("base", "quad", 4096): "eval_kernel_quad_int8_batch4096.md", ("base", "octo", 256): "duo_kernel_solo_int8_batch256.md",
             ("stress", "octo", 16384): "board_kernel_octo_512_int8_batch16384.md"}
    for key, name in where.items():
        assert key in bench.MEASURED_TRAFFIC_BYTES and name in text, key
    assert "0.445e9" in text["duo_kernel_int8_batch4096.md"] and bench.MEASURED_TRAFFIC_BYTES[("base", "duo", 4096)] == 0.445e9
    assert "0.78e9" in text["board_kernel_twin_int8_batch4096.md"] and bench.MEASURED_TRAFFIC_BYTES[("base", "twin", 4096)] == 0.78e9
    assert "5.938e8" in text["duo_kernel_int8_batch4096.md"] and bench.MEASURED_VALU_INSTS[("base", "duo", 4096)] == 5.938e8
    assert "5.513e8" in text["board_kernel_twin_int8_batch4096.md"] and bench.MEASURED_VALU_INSTS[("base", "twin", 4096)] == 5.513e8


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--steps", "5", "--warmup", "2", "--cpu-batch", "16"],
                         capture_output=True, text=True, timeout=400)
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [l for l in run.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    assert d["metric"] == "network evals/sec at batch 4096 int8 on 1 MI355X" and d["unit"] == "evals/s"
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["higher_is_better"] is True
    assert d["dtype"] == "int8" and d["data"] == "synthetic" and d["vs_baseline"] is None and d["scaling"] == "weak"
    assert set(d["config"]) == {"workload"} and "batch 4096" in d["config"]["workload"] and "kernel duo" in d["config"]["workload"]
    assert abs(d["value"] - 4096 / (d["ms_per_step"] * 1e-3)) < 1e-6 * d["value"]
    r = d["roofline"]
    assert r["bound"] == "mfma" and r["unit"] == "TOP/s" and r["peak"] == 5000.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-12
    assert abs(r["achieved"] - r["ops_per_launch"] / (r["kernel_ms"] * 1e-3) / 1e12) < 1e-6 * r["achieved"]
    assert r["ops_per_launch"] == 4096 * 402_653_184 and r["traffic"] > 0
    assert 0.5 * r["peak"] < r["measured_mfma_rate"] < 1.1 * r["peak"]
    assert d["value"] > 1.0e6          # a sanity bound, far below what the kernel measures (2.4-2.5 M)
    assert "5 steps between two device synchronisations" in d["step_protocol"]
    # the step time contains the kernel time; on a device at steady clocks they are within a few percent
    assert 0.9 * r["kernel_ms"] < d["ms_per_step"] < 1.25 * r["kernel_ms"]
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["unit"] == "evals/s" and c["cores"] >= 1 and c["value"] > 0 and "batch 16" in c["sample"]
    assert c["physical_cores"] >= 1 and c["fp32"]["value"] > 0
    # every configuration is in the default line: the sweep, e4m3 and the 512-wide network
    assert [p["batch"] for p in d["sweep"]] == [64, 256, 1024, 4096, 16384, 65536] and "interleaved" in d["timing_protocol"]
    assert all(p["ms_min_max"][0] <= p["ms_per_launch"] <= p["ms_min_max"][1] for p in d["sweep"])
    assert 0.5 < r["valu_floor_ms"] < r["kernel_ms"] and "vector ALU" in r["limiter"]
    assert all(p["ms_per_launch"] > 0 and p["kernel"] in ("octo", "duo") for p in d["sweep"])
    e = d["e4m3"]
    assert e["batch"] == 4096 and abs(e["frac_fp16_peak_2.5PF"] - 2 * e["frac_fp8_peak_5.0PF"]) < 1e-9 and e["evals_per_s"] > 5e5
    st = d["stress"]
    assert st["batch"] == 16384 and st["kernel"] == "octo" and 0.05 < st["frac_int8_peak"] < 1.0
    par = d["parity"]
    assert par["bit_exact_vs_c_checker"] is True and par["masked_argmax_equal"] is True
    assert par["prior_space_vs_int8_emulation"]["max_abs"] < 1e-2 and par["prior_space_vs_int8_emulation"]["edge_set_differs"] == 0
    assert r["weight_stream"]["bytes_per_launch"] == 2048 * 6_455_296                 # two positions share a copy
    nb = d["neighbours"]                      # move generation in front of the evaluator, edge expansion behind it
    assert [p["batch"] for p in nb] == [256, 4096, 65536]
    assert all(0 < p["movegen_ms"] < p["chain_ms"] and 0 < p["expand_ms"] < p["chain_ms"] for p in nb)
    assert all(0 < p["movegen_frac_hbm"] < 1 and 0 < p["expand_frac_hbm"] < 1 for p in nb)
    assert r["weight_stream"]["achieved_TBps"] < 1.1 * r["weight_stream"]["stream_ceiling_TBps"] < 1.1 * r["weight_stream"]["l1_fill_nominal_TBps"]


@pytest.mark.gpu
def test_phase_profile_flag_adds_the_phases_of_the_selected_kernel():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--no-cpu", "--no-extras", "--batch", "256",
                          "--steps", "2", "--warmup", "1", "--phases"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr[-2000:]
    d = json.loads([l for l in run.stdout.splitlines() if l.strip()][-1])
    ph = d["phases"]
    assert ph["kernel"] == "octo" and ph["ticks_per_wavefront"]["total"] > 0
    parts = [v for k, v in ph["share_of_total"].items() if k != "sync_wait"]     # barrier time is inside the phases
    assert 0.95 < sum(parts) < 1.05 and 0.0 < ph["share_of_total"]["sync_wait"] < 0.5
