"""ctypes binding of include/lumen_hip.h (lumen_amd/lib/liblumen_hip.so).

Loading fails loudly when the library has not been built: there is no CPU
fallback anywhere in this package.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# LUMEN_HIP_LIB: another build of the same library (e.g. the stage-time build of the Makefile)
LIB_PATH = os.environ.get("LUMEN_HIP_LIB") or os.path.join(_HERE, "lib", "liblumen_hip.so")

OK, ERR_SHAPE, ERR_KV_OVERFLOW, ERR_ROPE_RANGE, ERR_EMBED_OOB, ERR_CACHE_COUNT, ERR_INVALID, ERR_HIP, \
    ERR_NO_DEVICE, ERR_UNSUPPORTED = range(10)
DTYPE_F32, DTYPE_BF16 = 0, 1
DECODE_EAGER, DECODE_GRAPH, DECODE_PERSISTENT = 0, 1, 2

STATUS_NAMES = {OK: "OK", ERR_SHAPE: "SHAPE", ERR_KV_OVERFLOW: "KV_OVERFLOW", ERR_ROPE_RANGE: "ROPE_RANGE",
                ERR_EMBED_OOB: "EMBED_OOB", ERR_CACHE_COUNT: "CACHE_COUNT", ERR_INVALID: "INVALID",
                ERR_HIP: "HIP", ERR_NO_DEVICE: "NO_DEVICE", ERR_UNSUPPORTED: "UNSUPPORTED"}


class LumenError(RuntimeError):
    """A non-zero status from the library; .status is the code (the reference panics instead)."""

    def __init__(self, status, message):
        super().__init__("lumen status %d (%s): %s" % (status, STATUS_NAMES.get(status, "?"), message))
        self.status = status


class SamplingStruct(C.Structure):  # lumen_sampling
    _fields_ = [("temperature", C.c_float), ("top_p", C.c_float), ("repetition_penalty", C.c_float),
                ("recent_window", C.c_int), ("max_gen", C.c_int), ("seed", C.c_uint64)]


class LlamaConfigStruct(C.Structure):
    _fields_ = [("vocab_size", C.c_int), ("hidden_size", C.c_int), ("intermediate_size", C.c_int),
                ("num_hidden_layers", C.c_int), ("num_attention_heads", C.c_int),
                ("num_key_value_heads", C.c_int), ("rms_norm_eps", C.c_float), ("max_seq_len", C.c_int),
                ("rope_theta", C.c_float), ("head_dim", C.c_int), ("qk_norm", C.c_int),
                ("tie_embeddings", C.c_int), ("weight_dtype", C.c_int)]


_vp, _f, _i = C.c_void_p, C.c_float, C.c_int
_pp = C.POINTER(C.c_void_p)

# name -> (restype, argtypes); every symbol declared in include/lumen_hip.h
SIGNATURES = {
    "lumen_last_error": (C.c_char_p, []),
    "lumen_version": (C.c_char_p, []),
    "lumen_ctx_create": (_i, [_i, _pp]),
    "lumen_ctx_destroy": (_i, [_vp]),
    "lumen_ctx_set_stream": (_i, [_vp, _vp]),
    "lumen_ctx_synchronize": (_i, [_vp]),
    "lumen_timer_start": (_i, [_vp]),
    "lumen_timer_stop": (_i, [_vp, C.POINTER(_f)]),
    "lumen_malloc": (_i, [_vp, C.c_size_t, _pp]),
    "lumen_free": (_i, [_vp, _vp]),
    "lumen_ctx_num_cus": (_i, [_vp, _vp]),
    "lumen_upload": (_i, [_vp, _vp, _vp, C.c_size_t]),
    "lumen_download": (_i, [_vp, _vp, _vp, C.c_size_t]),
    "lumen_copy_d2d": (_i, [_vp, _vp, _vp, C.c_size_t]),
    "lumen_matmul_f32": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i]),
    "lumen_gemv_f32": (_i, [_vp, _vp, _vp, _vp, _i, _i]),
    "lumen_gemv_bench": (_i, [_vp, _vp, C.c_size_t, _i, _i, _vp, _vp, _i, _i, _i, C.POINTER(_f)]),
    "lumen_gemm_f32": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "lumen_gemv_bf16w": (_i, [_vp, _vp, _vp, _vp, _i, _i]),
    "lumen_gemv_fused_f32": (_i, [_vp, _vp, _i, _vp, _vp, _i, _i, _vp, _f, _i, _vp]),
    "lumen_interleave_rows": (_i, [_vp, _vp, _vp, _vp, _i, C.c_size_t]),
    "lumen_gemv_kernel_name": (_i, [_i, _i, _i, _i, _i, _i, C.c_char_p, _i]),
    "lumen_gemm_bf16w": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i]),
    "lumen_rmsnorm_f32": (_i, [_vp, _vp, _vp, _vp, _i, _i, _f]),
    "lumen_silu_f32": (_i, [_vp, _vp, _vp, C.c_size_t]),
    "lumen_copy_f32": (_i, [_vp, _vp, _vp, C.c_size_t]),
    "lumen_add_f32": (_i, [_vp, _vp, _vp, _vp, C.c_size_t]),
    "lumen_mul_f32": (_i, [_vp, _vp, _vp, _vp, C.c_size_t]),
    "lumen_swiglu_f32": (_i, [_vp, _vp, _vp, _vp, C.c_size_t]),
    "lumen_embedding_f32": (_i, [_vp, _vp, _vp, _i, _i, _i, _vp]),
    "lumen_argmax_f32": (_i, [_vp, _vp, _i, C.POINTER(_i)]),
    "lumen_rope_create": (_i, [_vp, _i, _i, _f, _pp]),
    "lumen_rope_destroy": (_i, [_vp]),
    "lumen_rope_tables_download": (_i, [_vp, _vp, _vp]),
    "lumen_rope_forward_f32": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i]),
    "lumen_rope_1token_copy_f32": (_i, [_vp, _vp, _vp, _i, _i]),
    "lumen_kv_cache_create": (_i, [_vp, _i, _i, _i, _i, _pp]),
    "lumen_kv_cache_destroy": (_i, [_vp]),
    "lumen_kv_cache_reset": (_i, [_vp]),
    "lumen_kv_cache_len": (_i, [_vp, C.POINTER(_i)]),
    "lumen_kv_cache_set_len": (_i, [_vp, _i]),
    "lumen_kv_cache_ptrs": (_i, [_vp, _pp, _pp]),
    "lumen_kv_cache_update": (_i, [_vp, _vp, _vp, _i, _i]),
    "lumen_kv_cache_get_view": (_i, [_vp, _i, _vp, _vp]),
    "lumen_attn_decode_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _f, _i]),
    "lumen_attn_decode_static_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _f, _i]),
    "lumen_qkv_rope_append_f32": (_i, [_vp, _vp, _vp, _i, _vp, _i, _vp, _f, _vp, _i]),
    "lumen_attn_decode_prerotated_f32": (_i, [_vp, _vp, _vp, _i, _f]),
    "lumen_attn_prefill_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _f, _i]),
    "lumen_llama_create": (_i, [_vp, C.POINTER(LlamaConfigStruct), _pp]),
    "lumen_llama_destroy": (_i, [_vp]),
    "lumen_llama_set_param": (_i, [_vp, C.c_char_p, _vp, _i, C.POINTER(C.c_int64), _i]),
    "lumen_llama_load_safetensors": (_i, [_vp, C.c_char_p, C.POINTER(_i), C.POINTER(_i)]),
    "lumen_sample_top_p_f32": (_i, [_vp, _i, _f, _f, _f, _vp, _i, _f, C.POINTER(C.c_int32)]),
    "lumen_rand01": (_f, [C.POINTER(C.c_uint64)]),
    "lumen_llama_generate_turn": (_i, [_vp, _vp, _i, _vp, _i, _vp, _vp, _i, _vp, _i, C.POINTER(_i)]),
    "lumen_llama_get_config": (_i, [_vp, _vp]),
    "lumen_safetensors_find": (_i, [C.c_char_p, C.c_char_p, C.POINTER(_i), C.POINTER(C.c_int64), C.POINTER(_i),
                                    C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "lumen_llama_forward": (_i, [_vp, _vp, _i, _vp, _i]),
    "lumen_llama_decode_greedy": (_i, [_vp, _i, _i, _vp, _vp]),
    "lumen_llama_decode_profile": (_i, [_vp, _i, _i, C.POINTER(C.c_double), C.POINTER(_i), _i]),
    "lumen_llama_set_decode_mode": (_i, [_vp, _i]),
    "lumen_llama_set_handover": (_i, [_vp, _i, C.c_int64, _i, _i, _i]),
    "lumen_llama_profile_kernel_name": (_i, [_vp, _i, C.c_char_p, _i]),
    "lumen_llama_get_decode_mode": (_i, [_vp, C.POINTER(_i)]),
    "lumen_llama_reset": (_i, [_vp]),
    "lumen_llama_kv_len": (_i, [_vp, C.POINTER(_i)]),
    "lumen_llama_set_kv_len": (_i, [_vp, _i]),
    "lumen_llama_cache_download": (_i, [_vp, _i, _vp, _vp]),
    "lumen_llama_cache_upload": (_i, [_vp, _i, _vp, _vp]),
    "lumen_llama_decode_bytes": (_i, [_vp, _i, C.POINTER(C.c_double)]),
    "lumen_decoder_layer_create": (_i, [_vp, C.POINTER(LlamaConfigStruct), _pp]),
    "lumen_decoder_layer_destroy": (_i, [_vp]),
    "lumen_decoder_layer_decode_f32": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
}


def load():
    if not os.path.exists(LIB_PATH):
        raise ImportError("%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                          "(hipcc --offload-arch=gfx950); lumen_amd has no CPU fallback" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the header and the library disagree
        fn.restype = res
        fn.argtypes = args
    return lib


GEMV_EPI_STORE, GEMV_EPI_RESIDUAL, GEMV_EPI_SWIGLU, GEMV_EPI_ARGMAX, GEMV_EPI_ROPE_QKV = range(5)

lib = load()


def gemv_kernel_name(num_cus, n, k, w_bf16, rmsnorm, epilogue):
    """The kernel instance the fused vector-matrix product launches for W [n, k] (host only, no GPU needed)."""
    buf = C.create_string_buffer(160)
    check(lib.lumen_gemv_kernel_name(int(num_cus), int(n), int(k), int(bool(w_bf16)), int(bool(rmsnorm)), int(epilogue), buf, 160))
    return buf.value.decode()


def check(status):
    if status != OK:
        raise LumenError(status, lib.lumen_last_error().decode("utf-8", "replace"))
