"""The benchmark's command-line contract: more than one GPU is refused with a message (the library
is a single-GPU kernel library), and on a GPU the default run prints one JSON line with the agreed
fields, short enough for a harness that keeps a few KB of output, and every case in a detail file."""
import json
import os
import subprocess
import sys

import pytest

from conftest import ROOT

BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode != 0
    assert "single-GPU" in out.stderr and out.stdout.strip() == ""


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline(tmp_path):
    detail_path = str(tmp_path / "detail.json")
    out = subprocess.run([sys.executable, BENCH, "--steps", "10", "--warmup", "2", "--cpu-rows", "256", "--detail", detail_path],
                         capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    # a harness that keeps only the tail of a run's output must still hold the whole line
    assert len(lines[0]) <= 4096 and len(out.stdout) + len(out.stderr) <= 8000
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "dense_fp32_gemm", "sweep", "summary"):
        assert key in line, key
    assert line["roofline"]["frac"] > 0.5 and line["cpu_baseline"]["value"] > 0
    sm = line["summary"]
    assert sm["digest_columns"] == ["cases", "min", "median", "max", "worst case"]
    assert sm["llm"]["frac_fp32_mfma_peak"][0] == 9 and sm["ragged"]["frac_fp32_mfma_peak"][0] == 9
    assert sm["decode"]["cold_frac_hbm"][0] == 16 and 0 < sm["decode"]["cold_frac_hbm"][3] <= 1.0
    assert "hot_gbs" in sm["decode"] and "hot_frac_hbm" not in sm["decode"]
    assert 0 < sm["compress_frac_hbm"][3] <= 1.0 and 0 < sm["decompress_frac_hbm"][3] <= 1.0
    assert sm["dispatch"]["cases"] == 12
    assert sm["sweep100_speedup_vs_dense"]["columns"][0] == "mean" and sm["sweep100_speedup_vs_dense"]["0.5"][0] > 1.5
    d = json.load(open(detail_path))
    assert all(d[k] == line[k] for k in ("value", "ms_per_step", "roofline", "cpu_baseline", "config"))
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 10 and d["warmup"] == 2 and d["vs_baseline"] is None
    assert d["dtype"] == "f32" and "workload" in d["config"]
    r = d["roofline"]
    assert r["bound"] == "mfma" and r["peak"] == 157.3 and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert abs(d["value"] - 2.0 * 4096 ** 2 * 2048 / (d["ms_per_step"] * 1e-3) / 1e12) < 0.01 * d["value"]
    c = d["cpu_baseline"]
    assert c["kind"] in ("reference", "port") and c["cores"] >= 1 and c["value"] > 0
    assert c["gpu_vs_cpu_scaled_max_error"] <= 1e-4
    assert set(d["sweep"]) == {"2:4", "3:8", "2:8", "1:8"}
    # every baseline workload is timed in the same run
    assert r["traffic_source"].startswith("profiles/") and r["traffic"] > r["algorithmic_bytes"] > 0
    assert r["kernel"].startswith("spmm_direct_kernel<32,16,4,1,")
    cfg = d["configs"]
    assert len(cfg["llm"]) == 9 and all(x["kernel"] == "mfma" and x["speedup_vs_dense"] > 1 for x in cfg["llm"])
    assert all(0.9 * x["ms"] < x["ms_b_from_hbm"] < 1.5 * x["ms"] for x in cfg["llm"])
    assert len(cfg["ragged"]) == 9 and cfg["ragged"][8]["rows_apart"] == 32 and all(x["kernel"] == "mfma" and 0.5 < x["frac_fp32_mfma_peak"] < 1 for x in cfg["ragged"])
    assert all(0.9 * x["ms"] < x["ms_b_from_hbm"] < 1.5 * x["ms"] for x in cfg["ragged"])
    assert cfg["ragged"][0]["waves_along_k"] == [128, 8] and cfg["ragged"][1]["waves_along_k"] == [64, 8]
    assert cfg["ragged"][2]["tile_wave_sets"] == 2 and cfg["ragged"][5]["tile_wave_rows"] == 256
    assert len(cfg["decode"]) == 16
    for x in cfg["decode"]:
        assert x["kernel"] == "decode" and x["kernel_reference_layout"] == "skinny"
        for mode in ("cold", "cold_stream_hint", "cold_reference_layout"):
            assert 0 < x[mode]["frac_hbm"] <= 1.0 and x[mode]["us"] > 0
        for mode in ("hot", "hot_reference_layout"):   # served by the Infinity Cache: a rate, no HBM fraction
            assert "frac_hbm" not in x[mode] and x[mode]["gbs"] > 0 and x[mode]["served_by"] == "infinity cache"
    assert len(cfg["decode_llm"]) == 9
    for x in cfg["decode_llm"]:
        assert x["kernel"] == "decode" and x["hot_split"]["us"] > 0 and x["cold_split"]["us"] > 0
    assert len(cfg["decode_wide"]) == 8 and all(x["kernel"] in ("decode", "mfma") and x["M"] in (48, 64) for x in cfg["decode_wide"])
    assert [x["pattern"] for x in cfg["fine"]][:4] == ["4:32", "8:32", "16:32", "2:4"] and cfg["fine"][3]["vec_len"] == 4
    assert cfg["fine"][-1]["pattern"] == "32:32" and cfg["fine"][-1]["kernel"] == "mfma"
    assert len(cfg["launch_constant"]) == 3 and len(cfg["compress"]) == 12 and len(cfg["rowmajor"]) == 5
    for x in cfg["compress"]:
        for name in ("compress", "decompress"):
            assert 0 < x[name]["frac_hbm"] <= 1.0 and "frac_hbm" not in x[name + "_hot"]
    for x in d["preprocess"]:
        assert x["host_pointer_dropin_wall_ms"] > 0 and x["cpu_restatement_wall_ms"] > 0
        assert x["device_reference_sequence_ms"] > 0
    for k, v in cfg["sweep100"]["by_sparsity"].items():
        assert len(v["rows"]) == 100 and v["mean_speedup_vs_dense"] > 0.7 / (1.0 - float(k))
    assert len(d["dispatch"]["shapes"]) == 12 and d["dispatch"]["mean_ratio"] < 1.1
    assert d["device"]["compute_units"] > 0 and d["device"]["dies"] > 0


@pytest.mark.gpu
def test_parts_can_be_selected(tmp_path):
    detail_path = str(tmp_path / "detail.json")
    out = subprocess.run([sys.executable, BENCH, "--steps", "5", "--warmup", "1", "--only", "fine", "--cpu-rows", "0",
                          "--fine-cases", "16:32x32,2:4x4", "--detail", detail_path],
                         capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr
    line = json.loads(out.stdout.strip())
    assert list(line["summary"]) == ["digest_columns", "fine_frac_fp32_mfma_peak"] and line["cpu_baseline"] is None and line["sweep"] == {}
    d = json.load(open(detail_path))
    assert list(d["configs"]) == ["fine"] and len(d["configs"]["fine"]) == 2 and d["dispatch"] is None
    bad = subprocess.run([sys.executable, BENCH, "--only", "nonsense"], capture_output=True, text=True, timeout=120)
    assert bad.returncode != 0 and "unknown part" in bad.stderr


def test_the_printed_line_stays_short_whatever_the_parts_hold():
    """The digests of the printed line are built from every part's rows; with rows of the real
    shape (long case names, wide numbers) for every part the line must stay under 4 KB, and the
    headline fields must survive the last-resort truncation."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_module", BENCH)
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    shape = {"M": 8192, "K": 11008, "Ncols": 14336, "pattern": "12:32"}
    rate = lambda hbm: {"us": 12345.67, "gbs": 7999.0, **({"frac_hbm": 0.999} if hbm else {"served_by": "infinity cache"})}
    decode_row = dict(shape, **{m[0]: rate(m[3]) for m in bench.DECODE_MODES})
    configs = {
        "llm": [dict(shape, frac_fp32_mfma_peak=0.999, speedup_over_ideal=1.234)] * 9,
        "ragged": [dict(shape, frac_fp32_mfma_peak=0.999)] * 9,
        "decode": [decode_row] * 16, "decode_llm": [decode_row] * 9, "decode_wide": [decode_row] * 8,
        "fine": [{"pattern": "16:32", "vec_len": 32, "frac_fp32_mfma_peak": 0.999}] * 8,
        "launch_constant": [{"pattern": "16:32", "constant_us": 10.25}] * 3,
        "compress": [dict(shape, compress=rate(True), decompress=rate(True), plain_copy_of_the_dense_operand=rate(True))] * 12,
        "rowmajor": [dict(shape, overhead=0.211)] * 5,
        "sweep100": {"by_sparsity": {k: {"mean_speedup_vs_dense": 19.268, "min_speedup_vs_dense": 10.123,
                                         "a100_reference_mean_speedup": 6.34} for k in ("0.5", "0.625", "0.75", "0.875")}},
    }
    # fine and launch_constant are keyed by pattern in the digest: give them distinct keys
    configs["fine"] = [dict(r, pattern="%d:32" % (i + 1)) for i, r in enumerate(configs["fine"])]
    configs["launch_constant"] = [dict(r, pattern="%d:32" % (i + 1)) for i, r in enumerate(configs["launch_constant"])]
    preprocess = [{"pattern": "%d:32" % i, "vec_len": 32, "device_one_kernel_ms": 0.0085, "cpu_restatement_wall_ms": 0.832,
                   "cpu_reference_wall_ms": 0.664} for i in range(4)]
    dispatch = {"shapes": [0] * 12, "mean_ratio": 1.001, "worst_ratio": 1.013}
    summary = bench.summarize(configs, preprocess, dispatch)
    size = len(json.dumps(summary, separators=(",", ":")))
    assert size <= 2400, size   # the headline fields take about 1.6 KB of the 4 KB
    assert set(summary) >= {"llm", "ragged", "decode", "decode_llm", "decode_wide", "compress_frac_hbm", "dispatch"}
