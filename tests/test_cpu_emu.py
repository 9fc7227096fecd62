"""The persistent decode kernel's device code, run on the CPU.

tests/cpu_emu builds lumen_amd/csrc/decode_persistent_device.h for the host (one OS thread per GPU
thread, pthread barriers for workgroup barriers, lock-step shuffles) with AddressSanitizer and runs
greedy decode steps of small models against the CPU oracle: grid barrier, cross-barrier weight
prefetch, split-attention merge and fused arg-max execute exactly as written.  An out-of-bounds
access aborts the run; the logits must match the oracle within the f32 / bf16 tolerances.
"""
import os
import subprocess

import pytest

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpu_emu")
EXE = os.path.join(HERE, "build", "emu_decode")
CLANG = "/opt/rocm/lib/llvm/bin/clang++"


@pytest.fixture(scope="module")
def emu():
    if not os.path.exists(CLANG):
        pytest.skip("ROCm clang++ not present")
    subprocess.run(["make", "-C", HERE], check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    return EXE


#        H    I    V   Hq Hkv D   L  max_seq qk bf16 steps nblocks start_pos
CASES = [
    (96, 160, 411, 4, 2, 64, 2, 80, 1, 0, 3, 2, 19),      # Qwen3-like: decoupled head_dim, q/k norm, n_rep 2
    (128, 352, 300, 2, 1, 64, 2, 256, 0, 0, 2, 3, 130),   # two attention slices per KV head (pos > 128)
    (256, 96, 200, 2, 2, 128, 1, 64, 0, 1, 2, 2, 5),      # head_dim 128, MHA, bf16 weights (ragged K sweeps)
    (64, 176, 97, 8, 1, 64, 1, 32, 0, 0, 3, 2, 0),        # n_rep 8 from an empty cache
]


@pytest.mark.parametrize("case", CASES, ids=["qwen3", "two-slices", "d128-bf16", "nrep8-empty"])
def test_persistent_kernel_on_cpu_matches_oracle(emu, case):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", OMP_NUM_THREADS="2")
    r = subprocess.run([emu] + [str(x) for x in case], env=env, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-4000:]
    assert "pick_mismatches=0" in r.stdout
