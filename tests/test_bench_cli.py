"""The benchmark's command line, without a GPU: more than one GPU is refused with a message (this build measures one
GPU's share of the path), and the flags the driver passes are accepted by the parser."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], stdout=subprocess.PIPE,
                          stderr=subprocess.STDOUT, text=True, timeout=120, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = run("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert proc.returncode != 0
    assert "ONE GPU" in proc.stdout and "--gpus 1" in proc.stdout


def test_help_lists_the_driver_flags():
    proc = run("--help")
    assert proc.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--workload", "--no-cpu-baseline"):
        assert flag in proc.stdout


def test_traffic_figures_are_the_ones_in_the_committed_profiles():
    """bench.py prints `roofline.traffic` from a table of constants; each must be the figure the rocprofv3 summary it
    names arrives at (written there as digits in groups of three, then " B")."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_for_traffic", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    assert set(bench.TRAFFIC) == {"gemv", "gemm", "moe_t64"}
    for key, (nbytes, source) in bench.TRAFFIC.items():
        text = open(os.path.join(ROOT, source)).read()
        assert f"{nbytes:,}".replace(",", " ") + " B" in text, (key, nbytes, source)
