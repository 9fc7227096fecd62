"""The decode path's device code on the CPU: tests/cpu_emu builds lumen_amd/csrc against a stand-in for the HIP
runtime (GPU threads as fibers, workgroups one after the other) with AddressSanitizer and
UndefinedBehaviorSanitizer, and its test program holds the chained launches (all forms, one and several attention
workgroups per head, q/k norm, bf16), the gate|up -> down chain and the few-row product to the checker.  Every load
and store of those kernels is bounds-checked there: device allocations, static and dynamic LDS are exact-sized host
objects.  No GPU involved."""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpu_emu")
EXE = os.path.join(HERE, "build", "emu_test")


@pytest.fixture(scope="module")
def emu():
    subprocess.run(["make", "-C", HERE, "-j8"], check=True, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE)
    assert os.path.exists(EXE)
    return EXE


def test_decode_kernels_on_the_cpu_under_sanitizers_match_the_checker(emu):
    r = subprocess.run([emu], capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    assert "cpu emulation: all checks passed" in r.stdout
    for case in ("chain:", "sliced:", "qknorm:", "bf16:", "skinny:", "attn:", "layerop:", "shapes:"):
        assert case in r.stdout
    assert "ERROR" not in r.stderr and "runtime error" not in r.stderr, r.stderr[-3000:]


def test_the_harness_stops_a_write_past_a_device_array(emu):
    r = subprocess.run([emu, "selfcheck-oob"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "AddressSanitizer" in r.stderr and "heap-buffer-overflow" in r.stderr, r.stderr[-2000:]
    assert "went unnoticed" not in r.stderr
