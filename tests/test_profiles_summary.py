"""The rocprofv3 summariser (gemm_mmbo_amd/profiles.py, `python -m gemm_mmbo_amd.report summarise`) on two tiny output
trees in rocprofv3's CSV layout whose numbers are round by construction (tests/golden/make_rocprof_fixture.py says what
each figure must come out as).  Pure CPU: the summariser never touches a GPU."""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FIX = os.path.join(ROOT, "tests", "golden", "rocprof")
sys.path.insert(0, ROOT)

from gemm_mmbo_amd import profiles as P  # noqa: E402


def test_bench_case_reports_the_median_of_the_timed_dispatches_and_the_box_independent_ratio():
    text = P.summarise("gemm_x16_f16_8192", os.path.join(FIX, "bench_f16"))
    # 12 dispatches, the last 5 timed: 700..740 us -> median 720 us; 2 * 8192^3 flop / 720 us = 1527.1 TFLOP/s = 0.6108 of 2500
    assert "the TIMED ones are the last 5" in text
    assert re.search(r"median 720\.0 us\s+min 700\.0\s+max 740\.0\s+mean 720\.0\s+gap between consecutive dispatches: median 0\.0 us", text)
    assert "=> 1527.1 TFLOP/s" in text and "= 0.6108 of the 2500.0 TFLOP/s matrix peak" in text
    # the unsettled launches (900 us) only appear in the all-dispatch mean: (7 * 900 + 3600) / 12 = 825
    assert "all 12 dispatches: mean 825.0 us" in text
    # the program's own record and the same-session ceiling: 1527.1 / 1900 = 0.8037
    assert "median 723.4 us per launch (1520.0 TFLOP/s, frac 0.608)" in text
    assert "random operands (mmbo_probe_mfma_ceiling): 1900.0 TFLOP/s at 1900 MHz = 0.760 of peak;  kernel / ceiling = 0.8037" in text
    # counters: the first tenth of the dispatches (one, with a tripled GRBM_GUI_ACTIVE) is dropped
    assert "9 dispatches (all but the first tenth), mean duration under counter collection 800.0 us" in text
    assert "shader clock = GRBM_GUI_ACTIVE / 8 XCDs / duration = 2.00 GHz" in text
    assert "1024 SIMDs) = 75.0 %   (busy x clock / 2.4 GHz = 0.625 of the matrix peak)" in text
    assert "SQ_INSTS_VALU_MFMA_MOPS_F16 * 512 = 1.0995e+12 flop (algorithmic 1.0995e+12)" in text
    assert "L2 hit rate = TCC_HIT / (TCC_HIT + TCC_MISS) = 75.0 %" in text
    # FETCH_SIZE 400,000 KiB x 1024 x 2.00 (calibration: 128 MiB true, 65,536 KiB counted) = 819 MB; WRITE_SIZE x 1.00 = 154 MB
    assert "FETCH_SIZE = 65536 KiB => factor 2.00" in text and "fetched per launch = 819 MB (algorithmic 268 MB)" in text
    assert "WRITE_SIZE = 131072 KiB => factor 1.00" in text and "written per launch = 154 MB (algorithmic 134 MB)" in text
    # every command line names committed files only, with the program directly behind `--`
    for line in re.findall(r"command: (.*)", text):
        assert re.search(r" -- python3 <repo>/bench\.py --no-cpu --only f16", line), line


def test_the_traffic_line_is_the_one_bench_py_reads(tmp_path, monkeypatch):
    import bench
    text = P.summarise("gemm_x16_f16_8192", os.path.join(FIX, "bench_f16"))
    prof = tmp_path / "profiles"
    prof.mkdir()
    (prof / "gemm_x16_f16_8192.txt").write_text(text)
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))
    total, source = bench.profiled_traffic("f16", "MT256x256x32_WT128x128_W4_GSU01_DTL1_RING5_MFMA16x16x32_ACC")
    assert total == pytest.approx(8.192e8 + 1.536e8) and "gemm_x16_f16_8192.txt" in source
    total, source = bench.profiled_traffic("f16", "some_other_tile")
    assert total is None and "was taken on" in source


def test_shapes_case_cuts_the_trace_by_call_and_sums_the_launches_of_a_split_k_gemm():
    P.CASES["_fixture"] = dict(P.CASES["skinny_cfg4"])
    try:
        text = P.summarise("_fixture", os.path.join(FIX, "shapes"))
    finally:
        del P.CASES["_fixture"]
    a, b = text.split("s,N,N,1024,1024,1024,1,1,0:")
    # shape 1: 6 calls of (GEMM 10 us, reduction 2 us), the last 4 timed; the reduction starts 3 us after the GEMM ends
    assert len(re.findall(r"timed dispatches\s+4\s+median\s+10\.0 us", a)) == 1 and len(re.findall(r"timed dispatches\s+4\s+median\s+2\.0 us", a)) == 1
    assert "per GEMM 12.0 us -> 357.9 TFLOP/s = 0.1432 of the 2500.0 TFLOP/s matrix peak; 2971 GB/s algorithmic" in a
    assert "gap between consecutive dispatches: median 3.0 us" in a and "15.5 us (277.1 TFLOP/s" in a
    assert "MFMA busy cycles = 25.0 % of the kernel's duration at 2.4 GHz" in a
    assert "fetched 43.0 MB, written 3.1 MB" in a          # (20,000 + 1,000) KiB x 2.0; (2,000 + 1,000) KiB x 1.0
    assert "kernel / ceiling" not in a                     # an HBM-bound shape has no MFMA ceiling to stand against
    # shape 2: one kernel of 20 us back to back: 2 * 1024^3 / 20 us = 107.4 TFLOP/s; / 150 = 0.7158
    assert "per GEMM 20.0 us -> 107.4 TFLOP/s = 0.6826 of the 157.3 TFLOP/s matrix peak" in b
    assert "gap between consecutive dispatches: median 0.0 us" in b and "kernel / ceiling (random operands) = 0.7158" in b
    assert "MFMA busy cycles = 50.0 %" in b and "fetched 12.3 MB, written 4.2 MB" in b


def test_a_trace_that_does_not_match_the_programs_records_is_refused():
    tr = P.read_trace(os.path.join(FIX, "shapes", "trace"))
    recs = [r for r in P.read_json_lines(os.path.join(FIX, "shapes", "trace.stdout")) if "calls_total" in r]
    assert [len(t) for _, _, t in P.split_by_shape(tr, recs)] == [8, 4]
    recs[1] = dict(recs[1], calls_total=7)
    with pytest.raises(ValueError, match="12 GEMM calls of this library, the program's records account for 13"):
        P.split_by_shape(tr, recs)


def test_command_line_front_end_and_fixture_generator(tmp_path):
    out = tmp_path / "s.txt"
    r = subprocess.run([sys.executable, "-m", "gemm_mmbo_amd.report", "summarise", "gemm_x16_f16_8192", os.path.join(FIX, "bench_f16"),
                        "--summary", str(out)], cwd=ROOT, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert "=> 1527.1 TFLOP/s" in out.read_text()
    r = subprocess.run([sys.executable, "-m", "gemm_mmbo_amd.report", "cases"], cwd=ROOT, capture_output=True, text=True)
    assert r.returncode == 0 and "gemm_x16_f16_8192" in r.stdout and "skinny_cfg4" in r.stdout
    # the committed fixture is what its generator writes
    before = {}
    for d, _, files in os.walk(FIX):
        for f in files:
            before[os.path.join(d, f)] = open(os.path.join(d, f), "rb").read()
    src = open(os.path.join(ROOT, "tests", "golden", "make_rocprof_fixture.py")).read().replace(
        'HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "rocprof")', f'HERE = {str(tmp_path / "regen")!r}')
    (tmp_path / "gen.py").write_text(src)
    assert subprocess.run([sys.executable, str(tmp_path / "gen.py")], capture_output=True).returncode == 0
    for path, data in before.items():
        assert open(os.path.join(str(tmp_path / "regen"), os.path.relpath(path, FIX)), "rb").read() == data, path
