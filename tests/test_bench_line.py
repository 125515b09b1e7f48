"""bench.py's stdout line has to stay short enough for a reader that keeps only a tail of
stdout: the per-operation tables go to a file, the line keeps the contract's fields."""
import importlib.util
import json
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def _bench():
    spec = importlib.util.spec_from_file_location("ctmi_bench", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _canned(bench):
    """a full default-run result with every optional part present and long strings"""
    roofline = {"bound": "hbm", "kernel": "pq_decompress_vec_kernel" * 2, "operation": "x" * 200,
                "achieved": 6512.123456789, "peak": 8000.0, "unit": "GB/s", "frac": 0.814015432,
                "achieved_bytes_per_launch": 627048448.123, "traffic": 627200000.0,
                "traffic_unit": "y" * 100, "traffic_source": "profiles/" + "z" * 80,
                "avg_launch_ms": 0.0962912345, "launches_per_step": 28,
                "compress_GBs": 6534.5, "decompress_GBs": 6511.9, "compress_ms": 2.69, "decompress_ms": 2.70}
    cpu = {"value": 2.7730519097067843, "unit": "GB/s", "cores": 16, "host_cpu_count": 384, "kind": "port",
           "sample": "compress+decompress of " + " + ".join(["14336x4096"] * 28) + " bf16, median of 5",
           "sample_short": "compress+decompress of 28 of the workload's tensors (872415232 elements), median of 5",
           "seconds": 1.5828550200000108}
    ops = [{"name": "operation number %d " % i + "n" * 90, "kernel": "k" * 40, "GBs": 1234.56789,
            "frac_of_hbm_peak": 0.1543, "ms": 0.123456, "algorithmic_bytes": 10 ** 9,
            "for_comparison_only": False, "launches": 28} for i in range(30)]
    configs = {w: {"metric": "m" * 120, "value": 5509.123, "unit": "GB/s", "steps": 5,
                   "ms_per_step_gpu": 20.1, "roofline": dict(roofline), "operations": ops,
                   "mfma_utilisation": {"frac": 0.17712345, "kernel": "k" * 30}, "cpu_baseline": dict(cpu)}
               for w in bench.OTHER_WORKLOADS}
    return {
        "metric": "compress+decompress GB/s & % HBM roofline, Llama-3-8B-shaped W4A16 g128",
        "value": 6514.123456789, "unit": "GB/s", "n_gpus": 1, "steps": 20, "warmup": 3,
        "ms_per_step": 5.390702749999576, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16 (" + "d" * 100 + ")", "data": "synthetic",
        "config": {"workload": "llama3-8b-w4a16", "tensors": 224, "elements": 6979321856,
                   "group_size": 128, "algorithmic_bytes_per_step": 35114713088, "scales": "s" * 100, "seed": 0},
        "hbm_roofline_frac": 0.8142, "roofline": roofline, "parity": "p" * 300, "cpu_baseline": cpu,
        "configs": configs,
        "api_level": {"what": "w" * 300, "compress_model_ms": 4.894932000013341,
                      "decompress_model_ms": 4.101406000003749, "frac_of_hbm_peak": 0.48790287070046295,
                      "other_formats": {
                          "float-quantized": {"compress_model_ms": 3.35, "decompress_model_ms": 3.49,
                                              "frac_of_hbm_peak": 0.76612345, "what": "w" * 200},
                          "nvfp4-pack-quantized": {"compress_model_ms": 3.07, "decompress_model_ms": 2.98,
                                                   "frac_of_hbm_peak": 0.73912345}}},
    }


def test_stdout_line_is_short_and_complete(tmp_path):
    bench = _bench()
    out = _canned(bench)
    assert len(json.dumps(out)) > 20000  # the full result is what used to be printed
    text = bench.short_line(out, str(ROOT / "gpurun_out" / "bench_details.json"))
    assert "\n" not in text
    assert len(text) <= 1500, len(text)
    line = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["dtype"] == "bf16"
    assert line["config"]["workload"] == "llama3-8b-w4a16"
    for key in ("bound", "kernel", "achieved", "peak", "unit", "frac", "traffic", "avg_launch_ms",
                "launches_per_step", "achieved_bytes_per_launch"):
        assert key in line["roofline"], key
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in line["cpu_baseline"], key
    assert set(line["configs_frac"]) == set(bench.OTHER_WORKLOADS)
    whole, slowest = line["configs_frac"]["sparse"]
    assert abs(whole - 1e9 / 0.123456 / 1e6 / 8000.0) < 5e-3 and abs(slowest - 0.1543) < 1e-3  # three digits
    assert abs(line["api_level"]["frac_of_hbm_peak"] - 0.4879) < 1e-4
    assert line["api_level"]["float-quantized"] == 0.766 and line["api_level"]["nvfp4-pack-quantized"] == 0.739
    assert abs(line["roofline"]["frac"] - out["roofline"]["frac"]) < 1e-3


def test_emit_writes_details_and_prints_one_line(tmp_path, capsys):
    bench = _bench()
    out = _canned(bench)
    path = tmp_path / "sub" / "details.json"
    bench.emit(out, str(path))
    printed = capsys.readouterr().out
    assert printed.count("\n") == 1 and len(printed) <= 1501
    assert json.loads(path.read_text())["configs"]["sparse"]["operations"][3]["launches"] == 28
    # a null traffic figure stays in the line as null
    out["roofline"]["traffic"] = None
    assert json.loads(bench.short_line(out))["roofline"]["traffic"] is None
