"""The CPU-side C under AddressSanitizer and UndefinedBehaviorSanitizer: `make -C oracle asan` builds oracle/sanitize_main.c
with the oracle and the host code of the product that needs no GPU (tables, fingerprints, every skeleton setter, the weight
file layout and the saved-array naming) and runs it; any report makes the run fail."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpu_side_c_is_clean_under_asan_and_ubsan():
    proc = subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "-B", "asan"], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-4000:]
    assert "sanitizer run clean" in proc.stdout
    assert "ERROR: AddressSanitizer" not in proc.stderr and "runtime error" not in proc.stderr
