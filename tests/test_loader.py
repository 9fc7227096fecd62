"""safetensors loading (src/loader.rs:10-80).  The files are written by the `safetensors` package, the same
container format the reference reads through the crate of that name; the library's own reader must find
every tensor where that package put it, and a model loaded from a file must equal one loaded tensor by tensor."""
import ctypes as C
import json
import struct

import numpy as np
import pytest

from lumen_amd import _lib, synth
from lumen_amd._lib import check, lib

st_numpy = pytest.importorskip("safetensors.numpy")

CFG = dict(vocab_size=300, hidden_size=64, intermediate_size=176, num_hidden_layers=2, num_attention_heads=4,
           num_key_value_heads=2, rms_norm_eps=1e-5, max_seq_len=48, rope_theta=10000.0)


def find(path, name):
    dtype, ndim = C.c_int(), C.c_int(8)
    shape = (C.c_int64 * 8)()
    b, e = C.c_uint64(), C.c_uint64()
    check(lib.lumen_safetensors_find(str(path).encode(), name.encode(), C.byref(dtype), shape, C.byref(ndim), C.byref(b), C.byref(e)))
    return dtype.value, tuple(shape[:ndim.value]), b.value, e.value


def header_of(path):
    raw = open(path, "rb").read()
    n = struct.unpack("<Q", raw[:8])[0]
    return json.loads(raw[8:8 + n]), raw[8 + n:]


def test_header_lookup_matches_the_file_written_by_the_safetensors_package(tmp_path):
    params = dict(synth.make_params(CFG, seed=5))
    p = tmp_path / "m.safetensors"
    st_numpy.save_file(params, str(p), metadata={"format": "pt", "note": 'quote " and {brace}'})
    hdr, data = header_of(p)
    for name, a in params.items():
        dtype, shape, b, e = find(p, name)
        assert dtype == _lib.DTYPE_F32 and shape == a.shape
        assert [b, e] == hdr[name]["data_offsets"]
        assert np.array_equal(np.frombuffer(data[b:e], np.float32).reshape(a.shape), a)
    with pytest.raises(_lib.LumenError) as err:
        find(p, "model.layers.9.mlp.up_proj.weight")
    assert err.value.status == _lib.ERR_INVALID
    with pytest.raises(_lib.LumenError):
        find(tmp_path / "absent.safetensors", "x")


def test_other_dtypes_and_damaged_files(tmp_path):
    p = tmp_path / "h.safetensors"
    st_numpy.save_file({"a": np.ones((2, 3), np.float16), "b": np.arange(4, dtype=np.int64)}, str(p))
    assert find(p, "a")[0] == -1 and find(p, "a")[1] == (2, 3) and find(p, "b")[0] == -1
    raw = open(p, "rb").read()
    bad = tmp_path / "bad.safetensors"
    bad.write_bytes(raw[:5])
    with pytest.raises(_lib.LumenError):
        find(bad, "a")
    bad.write_bytes(struct.pack("<Q", 1 << 40) + raw[8:])
    with pytest.raises(_lib.LumenError):
        find(bad, "a")
    bad.write_bytes(raw[:8] + b"[" + raw[9:])
    with pytest.raises(_lib.LumenError):
        find(bad, "a")
    # a header whose unknown value nests deeper than any real file: refused, not recursed into without bound;
    # 40 levels are still read
    def with_metadata(depth):
        hdr = ('{"__metadata__":' + "[" * depth + "]" * depth + ',"a":{"dtype":"F32","shape":[1],"data_offsets":[0,4]}}').encode()
        return struct.pack("<Q", len(hdr)) + hdr + b"\0\0\0\0"
    bad.write_bytes(with_metadata(40))
    assert find(bad, "a")[1] == (1,)
    bad.write_bytes(with_metadata(200000))
    with pytest.raises(_lib.LumenError):
        find(bad, "a")


@pytest.mark.gpu
def test_model_loaded_from_a_file_equals_the_model_loaded_tensor_by_tensor(tmp_path):
    import torch
    import safetensors.torch as st_torch
    from lumen_amd.models import LlamaModel

    params = dict(synth.make_params(CFG, seed=6, std=0.1, gains_one=False))
    ids = synth.make_tokens(9, CFG["vocab_size"], seed=6)
    ref = LlamaModel(CFG)
    ref.load_params(params)
    want = ref.forward(ids, all_rows=True)

    p = tmp_path / "f32.safetensors"
    st_numpy.save_file(params, str(p))
    m = LlamaModel(CFG)
    assert m.load_safetensors(p) == (len(params), 0)
    assert np.array_equal(m.forward(ids, all_rows=True), want)

    # bf16 file into an f32 model: widened like half::bf16::to_f32 (loader.rs:58)
    bits = {k: synth.bf16_round(v) for k, v in params.items()}
    pb = tmp_path / "bf16.safetensors"
    st_torch.save_file({k: torch.from_numpy(v.view(np.int16)).view(torch.bfloat16) for k, v in bits.items()}, str(pb))
    assert find(pb, "model.norm.weight")[0] == _lib.DTYPE_BF16
    m2, r2 = LlamaModel(CFG), LlamaModel(CFG)
    r2.load_params(bits)
    assert m2.load_safetensors(pb) == (len(params), 0)
    assert np.array_equal(m2.forward(ids, all_rows=True), r2.forward(ids, all_rows=True))

    # a parameter the file lacks is left as it is and counted (loader.rs:69-74)
    part = {k: v for k, v in params.items() if k != "lm_head.weight"}
    pp = tmp_path / "part.safetensors"
    st_numpy.save_file(part, str(pp))
    m3 = LlamaModel(CFG)
    m3.set_param("lm_head.weight", params["lm_head.weight"])
    assert m3.load_safetensors(pp) == (len(params) - 1, 1)
    assert np.array_equal(m3.forward(ids, all_rows=True), want)
    # ... and a weight nobody ever set is zero, not whatever the allocation held: all-zero logits here
    m4 = LlamaModel(CFG)
    assert m4.load_safetensors(pp) == (len(params) - 1, 1)
    assert not m4.forward(ids, all_rows=True).any()

    # unsupported dtype (loader.rs:67) and element-count mismatch (:44-46)
    ph = tmp_path / "f16.safetensors"
    st_numpy.save_file({k: v.astype(np.float16) for k, v in params.items()}, str(ph))
    with pytest.raises(_lib.LumenError) as e:
        LlamaModel(CFG).load_safetensors(ph)
    assert e.value.status == _lib.ERR_INVALID and "Unsupported dtype" in str(e.value)
    wrong = dict(params)
    wrong["model.norm.weight"] = np.ones(CFG["hidden_size"] + 1, np.float32)
    pw = tmp_path / "wrong.safetensors"
    st_numpy.save_file(wrong, str(pw))
    with pytest.raises(_lib.LumenError) as e:
        LlamaModel(CFG).load_safetensors(pw)
    assert e.value.status == _lib.ERR_SHAPE and "Shape mismatch for model.norm.weight" in str(e.value)
