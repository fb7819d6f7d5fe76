"""bench.py on a machine without a GPU: the flags of the driver's contract parse, more than one GPU is
refused with a message (this build runs on one), and the clock/power reader copes with missing files."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_without_a_gpu_it_says_so_instead_of_falling_back():
    import torch
    if torch.cuda.is_available():
        return
    r = _run("--steps", "1", "--warmup", "0", "--no-cpu")
    assert r.returncode == 3 and "no GPU" in r.stderr and r.stdout.strip() == ""


def test_clock_and_power_reader_returns_none_without_the_files():
    sys.path.insert(0, ROOT)
    import bench
    mhz, watts = bench.read_clock_and_power()
    assert mhz is None or mhz > 0
    assert watts is None or watts > 0
