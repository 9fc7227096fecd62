"""The C++ host layer (include/lumen.hpp): the reference's Rust surface for a compiled-language caller.

tests/host_cpp/test_host.cpp holds the checks themselves (every one through the C ABI, compared with the
CPU checker); this file compiles the header on its own, runs the device-free part here and the whole
program on the GPU.  The program is built by tests/host_cpp/Makefile (and by __graft_entry__.build()).
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HERE = os.path.join(ROOT, "tests", "host_cpp")
BINARY = os.path.join(HERE, "build", "test_host")


def _binary():
    if not os.path.exists(BINARY):
        subprocess.run(["make", "-C", HERE], check=True, stdout=subprocess.DEVNULL)
    return BINARY


def test_header_compiles_on_its_own(tmp_path):
    src = tmp_path / "only_header.cpp"
    src.write_text('#include "lumen.hpp"\nint main() { return lumen::is_no_grad() ? 1 : 0; }\n')
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only",
                    "-I", os.path.join(ROOT, "include"), str(src)], check=True)


def test_header_names_the_reference_surface():
    text = open(os.path.join(ROOT, "include", "lumen.hpp")).read()
    for name in ("class Tensor", "inline Tensor matmul", "struct Module", "class Linear", "class RMSNorm", "struct SiLU",
                 "class Embedding", "class RotaryEmbedding", "class KVCacheInner", "using KVCache", "class LlamaKVCache",
                 "class SelfAttention", "struct LlamaConfig", "class LlamaMLP", "class LlamaDecoderLayer",
                 "class LlamaModel", "struct ModelLoader", "load_llama_weights", "named_parameters", "init_kv_caches",
                 "reset_kv_caches", "forward_infer", "rope_1token_copy", "cos_sin_row_vec", "set_inference_mode",
                 "struct NoGradGuard", "sample_top_p"):
        assert name in text, name
    assert "oracle" not in text  # the host layer never reaches for the checker


def test_device_free_checks_pass():
    out = subprocess.run([_binary(), "--host-only"], capture_output=True, text=True, timeout=120)
    print(out.stdout)
    assert out.returncode == 0, out.stdout + out.stderr
    assert " 0 failed" in out.stdout


@pytest.mark.gpu
def test_host_layer_matches_the_checker_on_the_gpu():
    out = subprocess.run([_binary()], capture_output=True, text=True, timeout=300)
    print(out.stdout)
    assert out.returncode == 0, out.stdout + out.stderr
    assert " 0 failed" in out.stdout and "llama model and engine" in out.stdout
