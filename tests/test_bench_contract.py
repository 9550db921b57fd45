"""bench.py's command-line contract that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert p.returncode != 0
    assert "one GPU" in p.stderr and p.stdout.strip() == ""


def test_help_lists_the_contract_flags():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--op"):
        assert flag in p.stdout


def test_roofline_traffic_is_read_from_the_committed_profile():
    """bench.py takes roofline.traffic from the rocprofv3 --pmc summary under profiles/ (nothing re-typed in the script);
    the three workloads it is given for must parse, a missing section must give None and a reason."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    for section in ("decode", "prefill", "prefill_long"):
        nbytes, source = bench.profiled_traffic(section)
        assert nbytes is not None and 1e6 < nbytes < 1e11, (section, nbytes, source)
        assert "profiles/" in source and section in source
    nbytes, reason = bench.profiled_traffic("no_such_workload")
    assert nbytes is None and "no_such_workload" in reason
