"""CPU checks of bench.py's command-line contract (what can be checked without
a GPU): one GPU only, flags parse, and the constants it prices against."""
import os
import subprocess
import sys

from polarai_framework_amd import REPO_ROOT


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(REPO_ROOT, "bench.py"), *args],
                          capture_output=True, text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _bench("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout == ""


def test_help_lists_the_contract_flags():
    r = _bench("--help")
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup"):
        assert flag in r.stdout


def test_peaks_and_algorithmic_bytes():
    sys.path.insert(0, REPO_ROOT)
    import bench
    assert bench.HBM_PEAK_GBS == 8000.0 and bench.MFMA_FP32_PEAK_TFLOPS == 157.3
    assert bench.N_SWEEP == 1 << 26
    assert bench.BYTES_PER_ELEMENT["fadd"] == 12 and bench.BYTES_PER_ELEMENT["fsigmoid"] == 8
    assert bench.BYTES_PER_ELEMENT["ffill"] == 4 and bench.BYTES_PER_ELEMENT["ftranspose"] == 8
    assert set(bench.SWEEP) == {"fadd", "fmul", "fdivide", "fsigmoid", "fcopy", "ffill"}
