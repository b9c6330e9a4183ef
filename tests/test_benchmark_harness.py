"""The benchmark harness: shape table, options and statistics on the CPU; one tiny run on the GPU.

What it mirrors: the 20-shape table, the custom-shape options, the validation rules and the ops formula of
backends/_enflame/benchmarks/sage_attention_native_benchmark.py:70-78, :158-198, :447-455.
"""
import json
import os

import pytest

from baselinebenchmark_amd.benchmarks import sage_attention_benchmark as bench


def test_default_table_is_the_references_20_shapes_in_its_order():
    args = bench.build_parser().parse_args([])
    shapes = bench.configs(args)
    assert len(shapes) == 20 and len(set(shapes)) == 20
    assert shapes[0] == (1, 1024, 32, 32, 64, "float16")
    assert shapes[4] == (1, 16384, 32, 32, 64, "float16")
    assert shapes[5] == (1, 1024, 32, 32, 128, "float16")
    assert shapes[10] == (1, 1024, 32, 32, 64, "bfloat16")
    assert shapes[-1] == (1, 16384, 32, 32, 128, "bfloat16")
    assert {(b, t) for b, t, *_ in shapes} == {(1, 1024), (4, 1024), (1, 4096), (1, 8192), (1, 16384)}


def test_custom_shapes_and_validation():
    p = bench.build_parser()
    args = p.parse_args(["--custom-shapes", "--batch-size", "2", "--num-heads", "32", "--num-kv-heads", "8", "--head-dim", "128",
                         "--seq-lens", "512", "2048", "--dtype", "bfloat16"])
    bench.validate(args)
    assert bench.configs(args) == [(2, 512, 32, 8, 128, "bfloat16"), (2, 2048, 32, 8, 128, "bfloat16")]
    with pytest.raises(ValueError):
        bench.validate(p.parse_args(["--custom-shapes", "--num-heads", "6", "--num-kv-heads", "4"]))
    with pytest.raises(ValueError):
        bench.validate(p.parse_args(["--rep", "0"]))
    with pytest.raises(ValueError):
        bench.validate(p.parse_args(["--atol", "-1"]))
    with pytest.raises(SystemExit):
        p.parse_args(["--head-dim", "96"])
    with pytest.raises(ValueError):
        bench.validate(p.parse_args(["--blkk", "16", "--k-interleave", "4"]))
    bench.validate(p.parse_args(["--blkq", "32", "--q-interleave", "8", "--k-interleave", "4"]))


def test_ops_formula_and_statistics():
    assert bench.effective_ops(2, 32, 16384, 128, True) == 4398046511104.0      # BASELINE config 2
    assert bench.effective_ops(1, 32, 1024, 64, False) == 4 * 32 * 1024 * 1024 * 64
    s = bench.summarise([3.0, 1.0, 2.0, 100.0, 4.0])
    assert s["samples"] == 5 and s["median_ms"] == 3.0 and s["p99_ms"] == 100.0 and s["min_ms"] == 1.0 and s["mean_ms"] == 22.0
    s = bench.summarise([float(i) for i in range(1, 201)])
    assert s["p99_ms"] == 198.0 and s["median_ms"] == 100.5


@pytest.mark.gpu
@pytest.mark.sage_attention
def test_tiny_run_gates_then_times_and_writes_a_result_file(tmp_path):
    args = bench.build_parser().parse_args(["--custom-shapes", "--path", "both", "--batch-size", "1", "--num-heads", "4",
                                            "--num-kv-heads", "2", "--head-dim", "64", "--seq-lens", "256", "--warmup", "1",
                                            "--rep", "3", "--results-dir", str(tmp_path)])
    rows = bench.benchmark(args)
    assert [r["path"] for r in rows] == ["core", "e2e"]
    for r in rows:
        assert r["status"] == "PASS" and float(r["latency_ms"]) > 0 and float(r["gate_max_abs"]) < 3e-2 and r["samples"] == 3
    files = list(tmp_path.glob("sage_attention_mi355x_*.json"))
    assert len(files) == 1
    doc = json.loads(files[0].read_text())
    for key in ("backend", "device", "operator", "framework_version", "driver_version", "commit", "cases", "tolerance"):
        assert key in doc
    assert doc["cases"][0]["shape"] == [1, 4, 256, 64] and doc["cases"][0]["warmup"] == 1
    # upstream's per-thread granularities through the same gate and both paths
    args = bench.build_parser().parse_args(["--custom-shapes", "--path", "both", "--batch-size", "1", "--num-heads", "4",
                                            "--num-kv-heads", "2", "--head-dim", "128", "--seq-lens", "300", "--warmup", "1",
                                            "--rep", "2", "--blkq", "32", "--q-interleave", "8", "--k-interleave", "4", "--pv", "fp8",
                                            "--causal", "--results-dir", ""])
    rows = bench.benchmark(args)
    assert [r["status"] for r in rows] == ["PASS", "PASS"]


@pytest.mark.gpu
def test_hw_rate_microbenchmarks_run_and_are_plausible():
    """The micro-benchmarks behind the measured roofline denominators: every kind runs through the C ABI and the two
    MFMA instructions reach at least half of the datasheet rate from registers (they measure 80-95 % on the box)."""
    from baselinebenchmark_amd.benchmarks import hw_rates
    if not hw_rates.LIB_PATH.exists():
        pytest.skip("tool library absent (python -m baselinebenchmark_amd.build --tools)")
    rows = hw_rates.run(iters_mfma=500, iters_valu=2000)
    assert len(rows) == 3 * len(hw_rates.KINDS)
    best = {}
    for r in rows:
        assert r["seconds"] > 0
        if r["unit"] == "ops":
            best[r["kind"]] = max(best.get(r["kind"], 0.0), r["chip_TOPS"])
    assert best[0] > 2500 and best[1] > 2500, best
    assert best[3] <= best[0] * 1.15 and best[4] <= best[1] * 1.15, best   # feeding from LDS does not beat registers
    # co-execution: running the MFMA wavefront and the vector wavefront of a SIMD together takes at least as long as the
    # longer half alone and no longer than both in a row (a little slack for launch overhead on these short runs)
    co = hw_rates.run_coexec(iters=2000)
    assert len(co) == len(hw_rates.COEXEC_MFMA) * len(hw_rates.COEXEC_VALU)
    for r in co:
        assert r["both_s"] > 0.8 * max(r["mfma_alone_s"], r["valu_alone_s"]), r
        assert r["both_s"] < 1.3 * (r["mfma_alone_s"] + r["valu_alone_s"]), r
    # the attention kernel's tile period as an instruction mix: the pieces alone and together.  The matrix pipe alone
    # needs 2176 cycles per period (0.9 us at 2.4 GHz); everything together lies between the longest piece and their sum
    # (wide margins: these are short runs on whatever clock the box holds at that moment)
    rows = hw_rates.run_period(periods=1000)
    per = {r["parts"]: r["ns_per_period"] for r in rows}
    assert set(per) == {p for p, _ in hw_rates.PERIOD_PARTS} | {hw_rates.ROWS64}
    assert 700 < per[1] < 1600 and per[3] >= 0.9 * per[1] and per[11] >= 0.9 * per[3], per
    assert max(per[3], per[4]) * 0.9 <= per[15] <= 1.2 * (per[11] + per[4]), per
    # the same instructions on operand bits that toggle: not faster than on the regular pattern (beyond the noise of
    # these short runs), and not slower than the clock range of the part allows
    for r in rows:
        assert 0.8 * r["ns_per_period"] <= r["ns_per_period_random_operands"] <= 2.5 * r["ns_per_period"], r


@pytest.mark.gpu
def test_tile_timing_tool_reports_the_intervals_of_a_workgroup():
    """The instrumented twin of the library, loaded in its own process through SAGE_MI355X_LIB: every interval
    of a workgroup is positive and the main loop dominates a 4k-key causal tile."""
    import subprocess
    import sys
    from baselinebenchmark_amd.build import TIMING_LIB
    ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if not TIMING_LIB.exists():
        pytest.skip("timing build absent (python -m baselinebenchmark_amd.build --tools)")
    code = ("from baselinebenchmark_amd.benchmarks import tile_timing as t\n"
            "rows, tiles = t.measure(2, 4, 4096, 128, True, launches=2)\n"
            "line = t.timeline(2, 4, 4096, 128, True)\n"
            "import json; print(json.dumps({'rows': rows, 'tiles': tiles, 'timeline': line}))\n")
    env = dict(os.environ, SAGE_MI355X_LIB=str(TIMING_LIB))
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, cwd=ROOT, timeout=240)
    assert res.returncode == 0, res.stderr[-2000:]
    doc = json.loads([l for l in res.stdout.splitlines() if l.startswith("{")][-1])
    assert abs(doc["tiles"] - 17.0) < 1e-6          # 16 q-tiles of 256 rows: 2, 4, ..., 32 K tiles of 128 keys
    for name, vals in doc["rows"].items():
        if name == "request issue":
            assert len(vals) == 1 and vals[0] > 0
            continue
        if name == "raw Q wait":               # prologue: last request issued -> raw Q rows (and the first K tile) in LDS
            assert len(vals) == 1 and 0 < vals[0] < 1.0e5
            continue
        if name == "between workgroups":       # kernel wall time, workgroups per compute unit, cost beyond a workgroup's own stamps
            assert len(vals) == 3 and vals[0] > 0 and vals[1] > 0
            continue
        if name.endswith("phases"):          # main-loop phases per period: two phases and the waits at the two barriers
            assert len(vals) == 4 and all(v >= 0 for v in vals) and vals[0] > 0 and vals[2] > 0, (name, vals)
            continue
        assert len(vals) == 7 and all(v > 0 for v in vals), (name, vals)
        assert vals[4] > 0.5 * sum(vals), (name, vals)
    # the launch seen from the compute units: every workgroup recorded once, on some compute unit, inside the launch span;
    # 2 x 4 heads x 16 q-tiles with 2, 4, ..., 32 K tiles each
    line = doc["timeline"]
    assert line["workgroups"] == 128 and 1 <= line["compute_units"] <= 256
    assert abs(line["k_tiles_per_cu"][0] * line["compute_units"] - 8 * 272) < 1e-6
    assert line["inside_ns"][0] > 0 and line["gaps_ns"][1] >= 0 and line["after_last_ns"][1] == 0
    assert line["inside_ns"][2] <= line["span_ns"] and len(line["xcd_finish_before_end_ns"]) <= 8


@pytest.mark.gpu
def test_cpp_driver_calls_the_c_abi_directly():
    """sage_bench: a C++ program (no Python, no torch) that links libsage_mi355x.so, runs sage_sageattn and
    sage_sageattn_static on one stream with its own device buffers, gates the result and prints the table row."""
    import subprocess
    from baselinebenchmark_amd.build import CABI_BENCH
    if not CABI_BENCH.exists():
        pytest.skip("C++ driver absent (python -m baselinebenchmark_amd.build --tools)")
    for extra in ([], ["--static", "1"], ["--layout", "NHD", "--pv", "fp16", "--dtype", "fp16", "--kv-heads", "2"]):
        res = subprocess.run([str(CABI_BENCH), "--batch", "1", "--heads", "4", "--kv-heads", "4", "--seq", "1024", "--warmup", "2",
                              "--rep", "3", *extra], capture_output=True, text=True, timeout=120)
        assert res.returncode == 0, (extra, res.stdout, res.stderr)
        head, row = res.stdout.strip().splitlines()[-2:]
        cols = dict(zip(head.split("\t"), row.split("\t")))
        assert cols["gate"] == "PASS" and float(cols["latency_ms"]) > 0 and cols["backend"] == "mi355x_hip_int8_qk_fp8_fp16_pv"
