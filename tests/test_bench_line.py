"""The last stdout line of bench.py must stay a short, self-contained JSON record however many workloads the run
measured: a reader that keeps only the tail of stdout has to find it whole."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _canned(bench, n_rows):
    head = dict(tops=2391.1234567890123, ms_per_step=0.10059123456789012, tops_kernel=2444.9876543210987,
                us_kernel=98.37123456789012)
    cpu = dict(value=0.3456789012345678, unit="TOP/s", cores=16, kind="port",
               sample="first 2048 of 2048 rows of the headline workload (same weights), 0.7 s; output of the timed GPU "
                      "launches identical: True")
    others = []
    for i in range(n_rows):
        for name, extra in (("prefill_gemm", {}), ("bert_linear", dict(kind="deq")), ("decode_gemv", dict(M=1)),
                            ("decode_gemv", dict(M=16)), ("quantize_v2_scaled_qint8", {}), ("dequantize_scaled_qint8", {}),
                            ("requantize_int32_to_qint8", {})):
            others.append(dict(name=name, frac=0.4 + 0.001 * i, us_kernel=12.345678901234567, note="x" * 300, **extra))
    return head, cpu, others


def test_final_line_is_short_and_complete():
    bench = _bench()
    head, cpu, others = _canned(bench, 40)
    line = bench.summary_line(head, 20, 5, 222832901.80113044, cpu, others)
    text = json.dumps(line)
    assert len(text) < bench.MAX_LINE_BYTES <= 4096
    back = json.loads(text)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in back
    assert back["config"].keys() == {"workload"}
    assert set(back["roofline"]) >= {"bound", "achieved", "peak", "unit", "frac", "traffic"}
    assert abs(back["roofline"]["frac"] - back["roofline"]["achieved"] / back["roofline"]["peak"]) < 1e-12
    assert set(back["cpu_baseline"]) >= {"value", "unit", "cores", "kind", "sample"}
    assert "others" not in back
    assert back["targets"]["decode_gemv_m1_m4_frac_hbm_min"] == 0.4


def test_final_line_without_other_workloads_or_cpu_leg():
    bench = _bench()
    head, _, _ = _canned(bench, 0)
    line = bench.summary_line(head, 100, 20, None, None, [])
    text = json.dumps(line)
    assert len(text) < 4096 and json.loads(text)["cpu_baseline"] is None and line["targets"] == {}


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert proc.returncode != 0 and "one GPU" in proc.stderr
