"""The one stdout line of bench.py: short, parseable, with the roofline and CPU-baseline objects (no GPU needed)."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_headline_is_short_and_parses():
    bench = _bench()
    tuples = ["decode_tiled:AqBMMA_8x2xtrue_16x16x8192_16x16x512_16x16x64_6",
              "decode_tiled:AqBMMA_8x2xtrue_16x16x4096_16x16x512_16x16x64_6",
              "decode_tiled:AqBMMA_8x2xtrue_16x16x24576_16x16x512_16x16x64_6"]
    line = bench.headline(70.95, 20, 5, 0.000784, 9, 0.3, "decode_tiled", tuples, 9, 9051563.4, 4.319, 0.19432, 16,
                          "3 passes over the same 9 GEMMs (12.4 s), oracle popcount GEMM with OpenMP",
                          plane_operand_tops=49.8, extra_file="gpurun_out/bench_extra.json",
                          figures={"traffic_bytes_per_launch": 9306992, "avg_dispatch_ns": 4843})
    assert "\n" not in line and len(line) < 4096
    d = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert "extra" not in d
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0
    assert abs(r["achieved"] - 9051563.4 / 4.319e-6 / 1e9) < 0.1
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-4
    assert r["traffic"] == 9306992
    assert abs(r["frac_kernel_trace"] - 9051563.4 / 4843e-9 / 1e9 / 8000.0) < 1e-4
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] == 16 and c["unit"] == "TOPS"
    assert d["config"]["workload"].startswith("BASELINE configs[1]")


def test_traffic_is_read_from_the_committed_profile_summary(tmp_path):
    bench = _bench()
    # the committed summaries name the kernel family the headline runs on
    fig = bench.profile_figures("decode_tiled")
    assert fig["traffic_bytes_per_launch"] > 8_000_000 and fig["avg_dispatch_ns"] > 1000
    assert bench.profile_figures("some_other_kernel") == {}
    # a summary with another figure changes what the line reports; a missing one gives null, never a stale literal
    (tmp_path / bench.PROFILE_SUMMARIES[0]).write_text("x\nbench.py reads: `kernel=decode_tiled traffic_bytes_per_launch=123`\n")
    assert bench.profile_figures("decode_tiled", str(tmp_path)) == {"traffic_bytes_per_launch": 123,
                                                                    "source": ["profiles/" + bench.PROFILE_SUMMARIES[0]]}
    line = bench.headline(1.0, 1, 0, 1.0, 9, 0.0, "decode", ["decode:X"], 9, 1e6, 5.0, 0.1, 1, "s", figures={})
    assert json.loads(line)["roofline"]["traffic"] is None
