"""ctypes binding of the CPU oracle (oracle/lumen_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py as the checker / reported CPU baseline.  The
shipped package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "build", "liblumen_oracle.so")

LO_OK, LO_ERR_SHAPE, LO_ERR_KV_OVERFLOW, LO_ERR_ROPE_RANGE, LO_ERR_EMBED_OOB, LO_ERR_CACHE_COUNT = range(6)


def build(force=False):
    """Compile the oracle with gcc (oracle/Makefile)."""
    cmd = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()
_f = C.POINTER(C.c_float)
_u16 = C.POINTER(C.c_uint16)


def _p(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"], (a.dtype, a.flags)
    return a.ctypes.data_as(_f)


def _sig(name, res, *args):
    fn = getattr(_lib, name)
    fn.restype = res
    fn.argtypes = list(args)
    return fn


class KVCacheStruct(C.Structure):
    _fields_ = [("k", _f), ("v", _f), ("b", C.c_int), ("h_kv", C.c_int), ("max_seq", C.c_int),
                ("d", C.c_int), ("len", C.c_int)]


class LlamaConfigStruct(C.Structure):
    _fields_ = [("vocab_size", C.c_int), ("hidden_size", C.c_int), ("intermediate_size", C.c_int),
                ("num_hidden_layers", C.c_int), ("num_attention_heads", C.c_int),
                ("num_key_value_heads", C.c_int), ("rms_norm_eps", C.c_float),
                ("max_seq_len", C.c_int), ("rope_theta", C.c_float), ("head_dim", C.c_int),
                ("qk_norm", C.c_int), ("tie_embeddings", C.c_int)]


class LlamaLayerStruct(C.Structure):
    _fields_ = [(n, _f) for n in ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down", "input_norm",
                                  "post_norm", "q_norm", "k_norm")]


_sig("lo_set_threads", None, C.c_int)
_sig("lo_get_threads", C.c_int)
_sig("lo_gemv_f32", None, _f, _f, _f, C.c_int, C.c_int)
_sig("lo_gemm_f32", None, _f, _f, _f, C.c_int, C.c_int, C.c_int)
_sig("lo_matmul_f32", C.c_int, _f, _f, _f, C.c_int, C.c_int, C.c_int, C.c_int)
_sig("lo_rmsnorm_f32", None, _f, _f, _f, C.c_int, C.c_int, C.c_float)
_sig("lo_rope_table", None, _f, _f, C.c_int, C.c_int, C.c_float)
_sig("lo_rope_forward", C.c_int, _f, _f, _f, _f, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int)
_sig("lo_rope_1token_copy", C.c_int, _f, _f, _f, _f, C.c_int, C.c_int, C.c_int)
_sig("lo_silu_f32", None, _f, _f, C.c_long)
_sig("lo_add_f32", None, _f, _f, _f, C.c_long)
_sig("lo_mul_f32", None, _f, _f, _f, C.c_long)
_sig("lo_embedding_f32", C.c_int, _f, _f, C.c_int, C.c_int, C.c_int, _f)
_sig("lo_bf16_to_f32", None, _u16, _f, C.c_long)
_sig("lo_f32_to_bf16_rne", None, _f, _u16, C.c_long)
_sig("lo_argmax_f32", C.c_int, _f, C.c_int)
_sig("lo_sample_top_p", C.c_int, _f, C.c_int, C.c_float, C.c_float, C.c_float, C.POINTER(C.c_int), C.c_int, C.c_float)
_sig("lo_kv_cache_new", C.POINTER(KVCacheStruct), C.c_int, C.c_int, C.c_int, C.c_int)
_sig("lo_kv_cache_reset", None, C.POINTER(KVCacheStruct))
_sig("lo_kv_cache_free", None, C.POINTER(KVCacheStruct))
_sig("lo_attn_decode_f32", C.c_int, C.POINTER(KVCacheStruct), _f, _f, _f, _f, C.c_int, _f, _f, C.c_int,
     C.c_float, C.c_int)
_sig("lo_attn_prefill_f32", C.c_int, C.POINTER(KVCacheStruct), _f, _f, _f, _f, C.c_int, C.c_int, _f, _f,
     C.c_int, C.c_float, C.c_int)
_sig("lo_llama_new", C.c_void_p, C.POINTER(LlamaConfigStruct))
_sig("lo_llama_free", None, C.c_void_p)
_sig("lo_llama_set_globals", None, C.c_void_p, _f, _f, _f)
_sig("lo_llama_set_layer", None, C.c_void_p, C.c_int, C.POINTER(LlamaLayerStruct))
_sig("lo_llama_reset", None, C.c_void_p)
_sig("lo_llama_kv_len", C.c_int, C.c_void_p)
_sig("lo_llama_cache_k", _f, C.c_void_p, C.c_int)
_sig("lo_llama_cache_v", _f, C.c_void_p, C.c_int)
_sig("lo_llama_set_kv", C.c_int, C.c_void_p, C.c_int, _f, _f, C.c_int)
_sig("lo_llama_forward", C.c_int, C.c_void_p, _f, C.c_int, _f)


def set_threads(n):
    _lib.lo_set_threads(int(n))


def get_threads():
    return _lib.lo_get_threads()


def gemv(W, x):
    N, K = W.shape
    y = np.empty(N, np.float32)
    _lib.lo_gemv_f32(_p(W), _p(x), _p(y), N, K)
    return y


def gemm(A, W):
    M, K = A.shape
    N = W.shape[0]
    Cm = np.empty((M, N), np.float32)
    _lib.lo_gemm_f32(_p(A), _p(W), _p(Cm), M, N, K)
    return Cm


def matmul(a, w):
    """ops::matmul::matmul semantics: a [..., K] @ w[N, K]^T; returns (status, out)."""
    K_a = a.shape[-1]
    if w.ndim != 2:
        return LO_ERR_SHAPE, None
    N, K_w = w.shape
    M = a.size // max(K_a, 1)
    out = np.empty(a.shape[:-1] + (N,), np.float32)
    rc = _lib.lo_matmul_f32(_p(np.ascontiguousarray(a)), _p(w), _p(out), M, N, K_a, K_w)
    return rc, (out if rc == LO_OK else None)


def rmsnorm(x, w, eps):
    dim = x.shape[-1]
    rows = x.size // dim
    out = np.empty_like(x)
    _lib.lo_rmsnorm_f32(_p(x), _p(w), _p(out), rows, dim, float(eps))
    return out


def rope_table(dim, max_seq, theta):
    cos = np.empty((max_seq, dim), np.float32)
    sin = np.empty((max_seq, dim), np.float32)
    _lib.lo_rope_table(_p(cos), _p(sin), dim, max_seq, float(theta))
    return cos, sin


def rope_forward(x, cos, sin, offset):
    b, h, s, d = x.shape
    out = np.empty_like(x)
    rc = _lib.lo_rope_forward(_p(x), _p(out), _p(cos), _p(sin), b, h, s, d, offset, cos.shape[0])
    return rc, out


def rope_1token_copy(src, cos, sin, pos):
    dst = np.empty_like(src)
    rc = _lib.lo_rope_1token_copy(_p(src), _p(dst), _p(cos), _p(sin), src.shape[0], pos, cos.shape[0])
    return rc, dst


def silu(x):
    out = np.empty_like(x)
    _lib.lo_silu_f32(_p(x), _p(out), x.size)
    return out


def add(a, b):
    out = np.empty_like(a)
    _lib.lo_add_f32(_p(a), _p(b), _p(out), a.size)
    return out


def mul(a, b):
    out = np.empty_like(a)
    _lib.lo_mul_f32(_p(a), _p(b), _p(out), a.size)
    return out


def embedding(W, ids_f32):
    ids = np.ascontiguousarray(ids_f32, np.float32)
    out = np.empty(ids.shape + (W.shape[1],), np.float32)
    rc = _lib.lo_embedding_f32(_p(W), _p(ids), ids.size, W.shape[0], W.shape[1], _p(out))
    return rc, out


def bf16_to_f32(u16):
    u16 = np.ascontiguousarray(u16, np.uint16)
    out = np.empty(u16.shape, np.float32)
    _lib.lo_bf16_to_f32(u16.ctypes.data_as(_u16), _p(out), u16.size)
    return out


def f32_to_bf16(x):
    x = np.ascontiguousarray(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    _lib.lo_f32_to_bf16_rne(_p(x), out.ctypes.data_as(_u16), x.size)
    return out


def argmax(x):
    return _lib.lo_argmax_f32(_p(x), x.size)


def sample_top_p(logits, temperature, top_p, repetition_penalty, recent, r):
    """sample_top_p of src/main.rs:74-137 with the uniform draw r given."""
    logits = np.ascontiguousarray(logits, np.float32)
    rec = np.ascontiguousarray(recent, np.int32)
    return _lib.lo_sample_top_p(_p(logits), logits.size, float(temperature), float(top_p), float(repetition_penalty),
                                rec.ctypes.data_as(C.POINTER(C.c_int)), rec.size, float(r))


class KVCache:
    """KVCacheInner (self_attention.rs:24-44)."""

    def __init__(self, b, h_kv, max_seq, d):
        self._c = _lib.lo_kv_cache_new(b, h_kv, max_seq, d)
        self.shape = (b, h_kv, max_seq, d)

    def __del__(self):
        if getattr(self, "_c", None):
            _lib.lo_kv_cache_free(self._c)
            self._c = None

    @property
    def len(self):
        return self._c.contents.len

    def reset(self):
        _lib.lo_kv_cache_reset(self._c)

    @property
    def k(self):
        return np.ctypeslib.as_array(self._c.contents.k, shape=self.shape)

    @property
    def v(self):
        return np.ctypeslib.as_array(self._c.contents.v, shape=self.shape)


def attn_decode(cache, q3, k3, v3, cos, sin, scale, causal=True):
    """q3 [B,H,D], k3/v3 [B,Hkv,D] -> (status, out [B,1,H,D])."""
    b, h, d = q3.shape
    out = np.empty((b, 1, h, d), np.float32)
    rc = _lib.lo_attn_decode_f32(cache._c, _p(q3), _p(k3), _p(v3), _p(out), h, _p(cos), _p(sin),
                                 cos.shape[0], float(scale), int(causal))
    return rc, out


def attn_prefill(cache, q, k, v, cos, sin, scale, causal=True):
    """q [B,S,H,D], k/v [B,S,Hkv,D] -> (status, out [B,S,H,D])."""
    b, s, h, d = q.shape
    out = np.empty((b, s, h, d), np.float32)
    rc = _lib.lo_attn_prefill_f32(cache._c, _p(q), _p(k), _p(v), _p(out), s, h, _p(cos), _p(sin),
                                  cos.shape[0], float(scale), int(causal))
    return rc, out


class Llama:
    """LlamaModel (llama.rs:129-206) over a dict of HF-named f32 numpy weights
    (names as llama.rs:218-279).  Arrays are borrowed: the dict is kept alive."""

    def __init__(self, cfg, params):
        self.cfg = dict(cfg)
        c = LlamaConfigStruct(
            cfg["vocab_size"], cfg["hidden_size"], cfg["intermediate_size"], cfg["num_hidden_layers"],
            cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["rms_norm_eps"],
            cfg["max_seq_len"], cfg["rope_theta"], cfg.get("head_dim", 0) or 0,
            int(cfg.get("qk_norm", False)), int(cfg.get("tie_embeddings", False)))
        self._m = _lib.lo_llama_new(C.byref(c))
        self._params = params
        head = params["model.embed_tokens.weight"] if cfg.get("tie_embeddings") else params["lm_head.weight"]
        _lib.lo_llama_set_globals(self._m, _p(params["model.embed_tokens.weight"]),
                                  _p(params["model.norm.weight"]), _p(head))
        null = C.cast(None, _f)
        for i in range(cfg["num_hidden_layers"]):
            pre = "model.layers.%d." % i
            g = lambda n: _p(params[pre + n])
            ls = LlamaLayerStruct(
                g("self_attn.q_proj.weight"), g("self_attn.k_proj.weight"), g("self_attn.v_proj.weight"),
                g("self_attn.o_proj.weight"), g("mlp.gate_proj.weight"), g("mlp.up_proj.weight"),
                g("mlp.down_proj.weight"), g("input_layernorm.weight"), g("post_attention_layernorm.weight"),
                g("self_attn.q_norm.weight") if cfg.get("qk_norm") else null,
                g("self_attn.k_norm.weight") if cfg.get("qk_norm") else null)
            _lib.lo_llama_set_layer(self._m, i, C.byref(ls))

    def __del__(self):
        if getattr(self, "_m", None):
            _lib.lo_llama_free(self._m)
            self._m = None

    def reset(self):
        _lib.lo_llama_reset(self._m)

    @property
    def kv_len(self):
        return _lib.lo_llama_kv_len(self._m)

    def cache_k(self, layer):
        cfg = self.cfg
        d = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
        return np.ctypeslib.as_array(_lib.lo_llama_cache_k(self._m, layer),
                                     shape=(1, cfg["num_key_value_heads"], cfg["max_seq_len"], d))

    def cache_v(self, layer):
        cfg = self.cfg
        d = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
        return np.ctypeslib.as_array(_lib.lo_llama_cache_v(self._m, layer),
                                     shape=(1, cfg["num_key_value_heads"], cfg["max_seq_len"], d))

    def set_kv(self, layer, k, v, length):
        """Fills a layer's cache with rows computed elsewhere (k, v [1, Hkv, max_seq, D]) and sets its length:
        the fields of KVCacheInner are public (self_attention.rs:24-31)."""
        k, v = np.ascontiguousarray(k, np.float32), np.ascontiguousarray(v, np.float32)
        cfg = self.cfg
        d = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
        assert k.shape == v.shape == (1, cfg["num_key_value_heads"], cfg["max_seq_len"], d)
        return _lib.lo_llama_set_kv(self._m, layer, _p(k), _p(v), int(length))

    def forward(self, ids):
        """ids: sequence of token ids (cast to f32 like main.rs:143-152).
        Returns (status, logits [S, V])."""
        ids = np.ascontiguousarray(ids, np.float32).reshape(-1)
        logits = np.empty((ids.size, self.cfg["vocab_size"]), np.float32)
        rc = _lib.lo_llama_forward(self._m, _p(ids), ids.size, _p(logits))
        return rc, logits
