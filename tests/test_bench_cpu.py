"""bench.py without a GPU: the argument contract the driver relies on, and that every recorded traffic figure names a
summary under profiles/ that exists, states the command that made it and carries the figure."""
import importlib.util
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert run.returncode != 0 and "one GPU" in run.stderr and run.stdout.strip() == ""


def test_recorded_traffic_points_at_summaries_that_hold_it():
    bench = _bench()
    for key, (fetch, write, source) in bench.RECORDED_COUNTERS.items():
        path = os.path.join(ROOT, source)
        assert os.path.isfile(path), (key, source)
        text = open(path).read()
        assert "rocprofv3 --pmc FETCH_SIZE" in text and "rocprofv3 --pmc WRITE_SIZE" in text and "bench.py --only" in text, source
        digits = re.sub(r"(?<=\d) (?=\d{3})", "", text)          # "98 503" as 98503
        assert re.search(rf"(?<!\d){fetch}(?!\d)", digits) and re.search(rf"(?<!\d){write}(?:\.0)?(?!\d)", digits), (key, fetch, write, source)
        assert bench.RECORDED_TRAFFIC[key][0] == (2 * fetch + write) * 1024


def test_every_workload_of_only_is_dispatched():
    bench = _bench()
    source = open(os.path.join(ROOT, "bench.py")).read()
    for name in bench.ONLY:
        assert f'"{name}": lambda' in source or name == "bf16", name
    assert len(bench.RULE_CHECK_SHAPES) >= 27 and len(bench.VENDOR_GRID) >= 27
