"""The final stdout line of bench.py must stay small enough to be read whole from the tail of a log: it is built
by bench.compact_result(), fed here with a fake record for every workload the benchmark knows."""
import json

import bench


def fake_record(key, i):
    hbm = not key.startswith(("gemm_i8_8192", "gemm_f8", "gemm_bf16_2048", "peak_mfma", "pipeline", "gemm_i8_512",
                              "gemm_i8_4000", "gemm_f32", "gemm_f64"))
    dtype = "i8" if "i8" in key else "f8" if "f8" in key else "bf16" if "bf16" in key else "f16" if "f16" in key else "u8"
    unit = "GB/s" if hbm else "TOP/s" if dtype == "i8" else "TFLOP/s"
    roof = dict(bound="hbm" if hbm else "mfma", achieved=4321.123456789 + i, peak=8000.0 if hbm else 5000.0, unit=unit,
                frac=0.540140432098765, traffic=47093862 if i % 3 == 0 else None, kernel="some_kernel<with, a, long, name>" * 2,
                algorithmic_bytes=45136896)
    return dict(workload=key, name="a description of the workload that is fairly long, as the real ones are " * 2, steps=20,
                warmup=5, calls_per_step=128, ms_per_step=1.337133713371337, event_ms_per_call=0.010444444444444, dtype=dtype,
                value=4300.987654321, unit=unit, roofline=roof, peak_kind="hbm" if hbm else dtype, buffers_rotated=8)


def test_final_line_is_compact_and_complete():
    records = {key: fake_record(key, i) for i, key in enumerate(bench.WORKLOADS)}
    records["cvt_f32_f8e4m3_8192sq"] = {"workload": "cvt_f32_f8e4m3_8192sq", "error": "x" * 500}
    cpu = dict(value=1.99, unit="GB/s", cores=1, kind="reference", sample="s" * 90, host_cpus=256,
               all_cores=dict(value=31.3, unit="GB/s", cores=16, sample="t" * 90))
    result = bench.compact_result(records[bench.HEADLINE], records, cpu, "AMD Instinct MI355X (gfx950:sramecc+:xnack-), 256 CUs, 2400 MHz")
    result["full_results"] = "gpurun_out/bench_full.json"
    line = json.dumps(result, separators=(",", ":"))
    assert len(line) < 6000, len(line)
    back = json.loads(line)
    for field in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                  "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "device"):
        assert field in back, field
    roof = back["roofline"]
    for field in ("bound", "achieved", "peak", "unit", "frac", "traffic", "measured_peak", "frac_of_measured", "configs"):
        assert field in roof, field
    assert set(roof["configs"]) == set(bench.CONFIG_TABLE)
    assert "error" in roof["configs"].pop("C4 cvt f32->E4M3")
    for label, row in roof["configs"].items():
        assert set(row) >= {"key", "us", "achieved", "unit", "frac", "frac_of_measured"}, label
    assert back["config"]["workload"] and "model" not in back["config"]


def test_every_table_row_names_a_workload():
    assert set(bench.CONFIG_TABLE.values()) <= set(bench.WORKLOADS)
    assert set(bench.MEASURED_PEAK_OF.values()) <= set(bench.WORKLOADS)
