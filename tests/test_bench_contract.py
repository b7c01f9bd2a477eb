"""bench.py's command line: what it must do without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode == 2
    assert "one GPU only" in r.stderr and r.stdout.strip() == ""


def test_help_names_the_contract_flags():
    r = _run("--help")
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--no-cpu-baseline", "--prefill-probe", "--pmc-probe", "--e2e-only"):
        assert flag in r.stdout


def test_per_unit_figures_of_the_workload():
    """The algorithmic bytes the roofline is priced with: K * N / 4 per call, 120 calls per step."""
    sys.path.insert(0, ROOT)
    import bench

    names = {"wqkv": (3840, 2560), "wo": (2560, 2560), "w13": (13824, 2560), "w2": (2560, 6912)}
    src = open(os.path.join(ROOT, "bench.py")).read()
    for name, (n, k) in names.items():
        assert name in src
    total = sum(n * k // 4 for n, k in names.values())
    assert total == 17367040 and 30 * total == 521011200  # per layer, per step
    assert hasattr(bench, "cpu_baseline") and hasattr(bench, "latency_floor") and hasattr(bench, "generation_latency")
