"""Host-side checks of bench.py that need no GPU: the byte and FLOP counts behind the roofline figures, the refusal
of more than one GPU, and that an exception in an optional section does not take the contract's line with it."""
import importlib.util
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def load_bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_algorithmic_bytes_and_flops_of_the_headline_configs():
    b = load_bench()
    # decode at 32k: K + V reads, the two appends, q, k, v and the output (2 KV groups, 32 heads, d = 128)
    assert b.decode_bytes_per_layer(32768) == 33554432 + 1024 + 16384 + 2048 + 16384 == 33590272
    # 8192-token chunk at 24576, unmasked as the reference computes it: 4 h d pairs
    assert b.prefill_flops_per_layer(8192, 24576, causal=False) == 4 * 32 * 128 * 8192 * 32768
    # 2048-token causal prompt from an empty cache: the lower triangle with its diagonal
    assert b.prefill_flops_per_layer(2048, 0, causal=True) == 4 * 32 * 128 * (2048 * 2049 // 2)


def test_traffic_figure_comes_from_the_committed_counter_summary():
    b = load_bench()
    text = open(os.path.join(ROOT, b.DECODE_TRAFFIC_PROFILE)).read()
    n = b.decode_traffic_bytes_per_launch()
    assert n is not None and f"traffic_bytes_per_launch: {n:,}" in text
    # read once plus the exchange of the partials: between the algorithmic bytes and 1.5 times them
    assert b.decode_bytes_per_layer(32768) <= n < 1.5 * b.decode_bytes_per_layer(32768)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_an_optional_section_records_its_exception_and_lets_the_run_go_on():
    b = load_bench()
    result = {"value": 1.0}
    with b.optional_section(result, "layer"):
        raise RuntimeError("the whole-layer timing failed")
    assert result["value"] == 1.0
    assert result["layer"] == {"error": "RuntimeError: the whole-layer timing failed"}
    with b.optional_section(result, "model"):
        result["model"] = {"ok": True}
    assert result["model"] == {"ok": True}
    try:
        with b.optional_section(result, "linear"):
            raise KeyboardInterrupt()
    except KeyboardInterrupt:
        pass
    else:
        raise AssertionError("only exceptions of the Exception family are absorbed")
