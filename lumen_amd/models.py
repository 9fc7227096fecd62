"""LlamaModel of the reference (src/models/llama.rs) on the GPU.

LlamaModel drives the fused model-level entry points (one HIP-graph replay
per decoded token).  LayeredLlamaModel composes the same network from the
layer classes, one C-ABI call per reference operator, exactly as
LlamaDecoderLayer::forward_infer does; it exists so that the operator-level
drop-ins are exercised end to end.
"""
import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _lib, synth
from ._lib import ERR_CACHE_COUNT, LumenError, check, lib
from .autograd import Tensor, default_ctx
from .layers import Embedding, KVCacheInner, Linear, RMSNorm, SelfAttention, SiLU


@dataclass
class LlamaConfig:
    """src/models/llama.rs:11-37 plus the fields the other benchmark shapes need."""
    vocab_size: int = 32000
    hidden_size: int = 2048
    intermediate_size: int = 5632
    num_hidden_layers: int = 22
    num_attention_heads: int = 32
    num_key_value_heads: int = 4
    rms_norm_eps: float = 1e-5
    max_seq_len: int = 2048
    rope_theta: float = 10000.0
    head_dim: int = 0
    qk_norm: bool = False
    tie_embeddings: bool = False
    weight_dtype: str = "f32"

    @staticmethod
    def from_dict(d):
        return LlamaConfig(**{k: v for k, v in d.items()})

    def as_dict(self):
        return dict(self.__dict__)


class LlamaModel:
    """llama.rs:129-280.  Caches live inside the model (init_kv_caches(1) happens at construction);
    init_kv_caches / reset_kv_caches keep the reference's call shape."""

    def __init__(self, config, ctx=None):
        if isinstance(config, dict):
            config = LlamaConfig.from_dict(config)
        self.config = config
        self.ctx = ctx or default_ctx()
        c = _lib.LlamaConfigStruct(
            config.vocab_size, config.hidden_size, config.intermediate_size, config.num_hidden_layers,
            config.num_attention_heads, config.num_key_value_heads, config.rms_norm_eps, config.max_seq_len,
            config.rope_theta, config.head_dim or 0, int(config.qk_norm), int(config.tie_embeddings),
            _lib.DTYPE_BF16 if config.weight_dtype == "bf16" else _lib.DTYPE_F32)
        h = C.c_void_p()
        check(lib.lumen_llama_create(self.ctx.handle, C.byref(c), C.byref(h)))
        self.handle = h

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            lib.lumen_llama_destroy(h)

    # -- weights ------------------------------------------------------------
    def set_param(self, name, array):
        """One tensor by HF name (llama.rs:218-279); f32 arrays or bf16 bits as uint16 (loader.rs:32-68)."""
        a = np.ascontiguousarray(array)
        dtype = _lib.DTYPE_BF16 if a.dtype == np.uint16 else _lib.DTYPE_F32
        if dtype == _lib.DTYPE_F32 and a.dtype != np.float32:
            a = a.astype(np.float32)
        shape = (C.c_int64 * a.ndim)(*a.shape)
        check(lib.lumen_llama_set_param(self.handle, name.encode(), a.ctypes.data, dtype, shape, a.ndim))

    def load_safetensors(self, path):
        """ModelLoader::load_llama_weights (loader.rs:10-80): returns (tensors set, parameters the file lacks)."""
        loaded, missing = C.c_int(), C.c_int()
        check(lib.lumen_llama_load_safetensors(self.handle, str(path).encode(), C.byref(loaded), C.byref(missing)))
        return loaded.value, missing.value

    def generate_turn(self, new_tokens, history=(), temperature=0.8, top_p=0.9, repetition_penalty=1.05,
                      recent_window=96, max_gen=200, seed=0, stop_ids=()):
        """One turn of the chat loop (main.rs:325-378; defaults = its parameters, :223-227): prefill
        new_tokens, then sample until a stop id / max_gen / the end of the cache.  Returns the new ids."""
        new = np.ascontiguousarray(new_tokens, np.int32)
        hist = np.ascontiguousarray(history, np.int32)
        stops = np.ascontiguousarray(stop_ids, np.int32)
        sp = _lib.SamplingStruct(temperature, top_p, repetition_penalty, recent_window, max_gen, seed)
        out = np.zeros(max(max_gen, 1), np.int32)
        n = C.c_int()
        check(lib.lumen_llama_generate_turn(self.handle, new.ctypes.data, new.size, hist.ctypes.data, hist.size,
                                            C.byref(sp), stops.ctypes.data, stops.size, out.ctypes.data, out.size,
                                            C.byref(n)))
        return out[:n.value].copy()

    def load_params(self, named):
        for name, a in (named.items() if hasattr(named, "items") else named):
            self.set_param(name, a)

    def named_parameter_shapes(self):
        return synth.param_shapes(self.config.as_dict())

    # -- caches ---------------------------------------------------------------
    def init_kv_caches(self, batch_size=1):  # llama.rs:161-169
        if batch_size != 1:
            raise LumenError(_lib.ERR_UNSUPPORTED, "batch-1 path only")
        self.reset_kv_caches()
        return [("model-owned", i) for i in range(self.config.num_hidden_layers)]

    def reset_kv_caches(self, caches=None):  # llama.rs:172-176
        check(lib.lumen_llama_reset(self.handle))

    @property
    def kv_len(self):
        n = C.c_int()
        check(lib.lumen_llama_kv_len(self.handle, C.byref(n)))
        return n.value

    def set_kv_len(self, length):
        """Back to an earlier cache length (KVCacheInner.len is a public field, self_attention.rs:28): the rows beyond
        it are overwritten by the steps that follow."""
        check(lib.lumen_llama_set_kv_len(self.handle, int(length)))

    def cache(self, layer):
        cfg = self.config
        d = cfg.head_dim or cfg.hidden_size // cfg.num_attention_heads
        shape = (1, cfg.num_key_value_heads, cfg.max_seq_len, d)
        k, v = np.empty(shape, np.float32), np.empty(shape, np.float32)
        check(lib.lumen_llama_cache_download(self.handle, layer, k.ctypes.data, v.ctypes.data))
        return k, v

    def set_cache(self, layer, k, v):
        """A layer's cache rows from host arrays [1, H_kv, max_seq, D] (public fields of KVCacheInner,
        self_attention.rs:24-31); set_kv_len then says how many rows are valid."""
        k, v = np.ascontiguousarray(k, np.float32), np.ascontiguousarray(v, np.float32)
        cfg = self.config
        d = cfg.head_dim or cfg.hidden_size // cfg.num_attention_heads
        assert k.shape == v.shape == (1, cfg.num_key_value_heads, cfg.max_seq_len, d)
        check(lib.lumen_llama_cache_upload(self.handle, int(layer), k.ctypes.data, v.ctypes.data))

    # -- forward ----------------------------------------------------------------
    def forward(self, input_ids, caches=None, _pos=0, all_rows=True):
        """llama.rs:181-206.  input_ids: token ids (any numeric dtype; they travel as f32 like
        main.rs:143-152).  Returns host logits [S, V] (all_rows) or [V] (last position only)."""
        if caches is not None and len(caches) != self.config.num_hidden_layers:  # llama.rs:182-188
            raise LumenError(ERR_CACHE_COUNT, "KV cache count mismatch: got %d, expected %d"
                             % (len(caches), self.config.num_hidden_layers))
        ids = np.ascontiguousarray(input_ids, np.float32).reshape(-1)
        s = ids.size
        out = np.empty((s, self.config.vocab_size) if all_rows else (self.config.vocab_size,), np.float32)
        check(lib.lumen_llama_forward(self.handle, ids.ctypes.data, s, out.ctypes.data, int(all_rows)))
        return out

    def decode_greedy(self, first_id, n, want_logits=False):
        """The generation loop of main.rs:340-378 with greedy picks, entirely on the GPU."""
        ids = np.empty(n, np.int32)
        logits = np.empty((n, self.config.vocab_size), np.float32) if want_logits else None
        check(lib.lumen_llama_decode_greedy(self.handle, int(first_id), n, ids.ctypes.data,
                                            logits.ctypes.data if want_logits else None))
        return (ids, logits) if want_logits else ids

    DECODE_MODES = {"eager": _lib.DECODE_EAGER, "graph": _lib.DECODE_GRAPH, "persistent": _lib.DECODE_PERSISTENT}

    def set_decode_mode(self, mode):
        """'graph' (HIP graph replay per token) or 'eager' (kernel by kernel); 'persistent' is refused
        (the library holds no such kernel)."""
        check(lib.lumen_llama_set_decode_mode(self.handle, self.DECODE_MODES[mode]))

    def set_handover(self, enable=-1, spin_limit=-1, pre_sleep=-1, poll_delay=-1, poll_gap=-1):
        """The chained launch of short caches: 0 separate launches, 1 attention -> o_proj, 2 q|k|v -> attention ->
        o_proj; and the limits and pauses of its waits (negative: unchanged)."""
        check(lib.lumen_llama_set_handover(self.handle, int(enable), int(spin_limit), int(pre_sleep), int(poll_delay),
                                           int(poll_gap)))

    @property
    def decode_mode(self):
        v = C.c_int()
        check(lib.lumen_llama_get_decode_mode(self.handle, C.byref(v)))
        return {n: k for k, n in self.DECODE_MODES.items()}[v.value]

    KERNEL_CLASSES = ("embedding", "norm_qkv_gemv", "attn_decode", "oproj_gemv", "norm_gateup_gemv", "down_gemv",
                      "norm_lmhead_gemv", "argmax", "attn_oproj_fused", "mlp_fused")

    def profile_kernel_name(self, kernel_class):
        """The kernel instance the last decode_profile launched for a class ('' if none)."""
        buf = C.create_string_buffer(160)
        check(lib.lumen_llama_profile_kernel_name(self.handle, self.KERNEL_CLASSES.index(kernel_class), buf, 160))
        return buf.value.decode()

    def decode_profile(self, first_id, n):
        """n greedy steps with every launch bracketed by HIP events: {class: (ms_sum, launches)}."""
        k = len(self.KERNEL_CLASSES)
        ms = (C.c_double * k)()
        cnt = (C.c_int * k)()
        check(lib.lumen_llama_decode_profile(self.handle, int(first_id), int(n), ms, cnt, k))
        return {name: (ms[i], cnt[i]) for i, name in enumerate(self.KERNEL_CLASSES)}

    def decode_bytes(self, length):
        b = C.c_double()
        check(lib.lumen_llama_decode_bytes(self.handle, int(length), C.byref(b)))
        return b.value


class LlamaMLP:
    """llama.rs:41-66: down(silu(gate(x)) * up(x)) as five separate operator calls."""

    def __init__(self, gate_w, up_w, down_w):
        self.gate_proj, self.up_proj, self.down_proj = Linear(gate_w), Linear(up_w), Linear(down_w)
        self.act = SiLU()

    def forward(self, x):
        gate = self.gate_proj.forward(x)
        gate_act = self.act.forward(gate)
        up = self.up_proj.forward(x)
        fused = gate_act * up
        return self.down_proj.forward(fused)


class LlamaDecoderLayer:
    """llama.rs:79-116 (forward_infer)."""

    def __init__(self, cfg, params, prefix, ctx):
        self.self_attn = SelfAttention(cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads,
                                       cfg.max_seq_len, cfg.rope_theta, True, ctx)
        for attr, name in (("w_q", "q_proj"), ("w_k", "k_proj"), ("w_v", "v_proj"), ("w_o", "o_proj")):
            setattr(self.self_attn, attr, Linear(Tensor.from_array_no_grad(params[prefix + "self_attn.%s.weight" % name], ctx)))
        t = lambda n: Tensor.from_array_no_grad(params[prefix + n], ctx)
        self.mlp = LlamaMLP(t("mlp.gate_proj.weight"), t("mlp.up_proj.weight"), t("mlp.down_proj.weight"))
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps, params[prefix + "input_layernorm.weight"], ctx)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_norm_eps,
                                                params[prefix + "post_attention_layernorm.weight"], ctx)

    def fuse(self):
        """Lays the weights out for the fused single-token operators: w_q | w_k | w_v rows one after the other,
        gate_proj / up_proj rows interleaved (device-to-device copies, once)."""
        a, ctx = self.self_attn, self.self_attn.ctx
        wq, wk, wv = a.w_q.weight, a.w_k.weight, a.w_v.weight
        k = wq.shape[1]
        self.w_qkv = Tensor.empty((wq.shape[0] + wk.shape[0] + wv.shape[0], k), np.float32, ctx)
        off = 0
        for w in (wq, wk, wv):
            check(lib.lumen_copy_d2d(ctx.handle, self.w_qkv.ptr + off, w.ptr, w.size * 4))
            off += w.size * 4
        g, u = self.mlp.gate_proj.weight, self.mlp.up_proj.weight
        self.w_gate_up = Tensor.empty((2 * g.shape[0], g.shape[1]), np.float32, ctx)
        check(lib.lumen_interleave_rows(ctx.handle, g.ptr, u.ptr, self.w_gate_up.ptr, g.shape[0], g.shape[1] * 4))
        self.fused = True

    def forward_token(self, x, cache):
        """forward_infer for S == 1 through the fused operators: five launches (llama.rs:104-116 with the leaves
        of :59-65 and self_attention.rs:106-108, :161-176, :183-303 folded as the decode step folds them)."""
        a, ctx = self.self_attn, self.self_attn.ctx
        h, d = a.n_head, a.head_dim
        hidden = x.shape[-1]
        q_rot = Tensor.empty((h * d,), np.float32, ctx)
        check(lib.lumen_qkv_rope_append_f32(cache.handle, a.rope.handle, self.w_qkv.ptr, 0, x.ptr, hidden,
                                            self.input_layernorm.weight.ptr, self.input_layernorm.eps, q_rot.ptr, h))
        attn = Tensor.empty((h * d,), np.float32, ctx)
        check(lib.lumen_attn_decode_prerotated_f32(cache.handle, q_rot.ptr, attn.ptr, h, a.scale))
        hbuf = Tensor.empty(x.shape, np.float32, ctx)
        check(lib.lumen_gemv_fused_f32(ctx.handle, a.w_o.weight.ptr, 0, attn.ptr, hbuf.ptr, hidden, h * d, None, 0.0,
                                       _lib.GEMV_EPI_RESIDUAL, x.ptr))
        inter = self.mlp.down_proj.weight.shape[1]
        act = Tensor.empty((inter,), np.float32, ctx)
        check(lib.lumen_gemv_fused_f32(ctx.handle, self.w_gate_up.ptr, 0, hbuf.ptr, act.ptr, 2 * inter, hidden,
                                       self.post_attention_layernorm.weight.ptr, self.post_attention_layernorm.eps,
                                       _lib.GEMV_EPI_SWIGLU, None))
        out = Tensor.empty(x.shape, np.float32, ctx)
        check(lib.lumen_gemv_fused_f32(ctx.handle, self.mlp.down_proj.weight.ptr, 0, act.ptr, out.ptr, hidden, inter,
                                       None, 0.0, _lib.GEMV_EPI_RESIDUAL, hbuf.ptr))
        return out, cache

    def forward_token_layer_op(self, x, cache, op):
        """forward_infer for S == 1 as ONE operator call (lumen_decoder_layer_decode_f32): the launches of the
        model-level decode step, three per layer where the chained launch covers the shape."""
        out = Tensor.empty(x.shape, np.float32, self.self_attn.ctx)
        check(lib.lumen_decoder_layer_decode_f32(op.handle, cache.handle, self.w_qkv.ptr, self.self_attn.w_o.weight.ptr,
                                                 self.w_gate_up.ptr, self.mlp.down_proj.weight.ptr,
                                                 self.input_layernorm.weight.ptr, self.post_attention_layernorm.weight.ptr,
                                                 None, None, x.ptr, out.ptr))
        return out, cache

    def forward_infer(self, x, cache, layer_op=None):
        if layer_op is not None and x.shape[0] == 1 and x.shape[1] == 1:
            return self.forward_token_layer_op(x, cache, layer_op)
        if getattr(self, "fused", False) and x.shape[0] == 1 and x.shape[1] == 1:
            return self.forward_token(x, cache)
        norm_x = self.input_layernorm.forward(x)
        attn_out, cache_out = self.self_attn.forward(norm_x, cache)
        h = x + attn_out
        norm_h = self.post_attention_layernorm.forward(h)
        mlp_out = self.mlp.forward(norm_h)
        return h + mlp_out, cache_out


class DecoderLayerOp:
    """The state a layer-level decode step needs besides weights and cache (lumen_decoder_layer): one serves all
    layers of a stack."""

    def __init__(self, config, ctx=None):
        if isinstance(config, dict):
            config = LlamaConfig.from_dict(config)
        self.ctx = ctx or default_ctx()
        c = _lib.LlamaConfigStruct(
            config.vocab_size, config.hidden_size, config.intermediate_size, config.num_hidden_layers,
            config.num_attention_heads, config.num_key_value_heads, config.rms_norm_eps, config.max_seq_len,
            config.rope_theta, config.head_dim or 0, int(config.qk_norm), int(config.tie_embeddings),
            _lib.DTYPE_BF16 if config.weight_dtype == "bf16" else _lib.DTYPE_F32)
        h = C.c_void_p()
        check(lib.lumen_decoder_layer_create(self.ctx.handle, C.byref(c), C.byref(h)))
        self.handle = h

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            lib.lumen_decoder_layer_destroy(h)


class LayeredLlamaModel:
    """LlamaModel::forward (llama.rs:181-206) composed operator by operator.  fused=True (default): a single
    token (S == 1) takes the fused operators -- five launches per layer, and the final norm rides on the lm_head
    product -- as the model-level decode step does; fused=False: one call per reference leaf, every time;
    layer_op=True: a single token takes ONE operator call per layer (lumen_decoder_layer_decode_f32: the chained
    launches of the model-level step, three per layer where they cover the shape)."""

    def __init__(self, config, params, ctx=None, fused=True, layer_op=False):
        if isinstance(config, dict):
            config = LlamaConfig.from_dict(config)
        if config.head_dim or config.qk_norm or config.tie_embeddings or config.weight_dtype != "f32":
            raise LumenError(_lib.ERR_UNSUPPORTED, "the layered model covers the reference's Llama shape only")
        self.config = config
        self.ctx = ctx or default_ctx()
        self.embed_tokens = Embedding(Tensor.from_array_no_grad(params["model.embed_tokens.weight"], self.ctx))
        self.layers = [LlamaDecoderLayer(config, params, "model.layers.%d." % i, self.ctx)
                       for i in range(config.num_hidden_layers)]
        self.norm = RMSNorm(config.hidden_size, config.rms_norm_eps, params["model.norm.weight"], self.ctx)
        self.lm_head = Linear(Tensor.from_array_no_grad(params["lm_head.weight"], self.ctx))
        self.fused = bool(fused) or bool(layer_op)
        self.layer_op = DecoderLayerOp(config, self.ctx) if layer_op else None
        if self.fused:
            for layer in self.layers:
                layer.fuse()

    def init_kv_caches(self, batch_size=1):
        c = self.config
        d = c.hidden_size // c.num_attention_heads
        return [KVCacheInner(batch_size, c.num_key_value_heads, c.max_seq_len, d, self.ctx)
                for _ in range(c.num_hidden_layers)]

    def reset_kv_caches(self, caches):
        for c in caches:
            c.reset()

    def forward(self, input_ids, caches, _pos=0):
        if len(caches) != len(self.layers):
            raise LumenError(ERR_CACHE_COUNT, "KV cache count mismatch: got %d, expected %d"
                             % (len(caches), len(self.layers)))
        ids = np.ascontiguousarray(input_ids, np.float32).reshape(1, -1)
        x = self.embed_tokens.forward(ids)
        for i, layer in enumerate(self.layers):
            x, caches[i] = layer.forward_infer(x, caches[i], self.layer_op)
        if self.fused and ids.shape[1] == 1:  # final norm + lm_head in one launch (llama.rs:202-205)
            w = self.lm_head.weight
            logits = Tensor.empty((1, 1, w.shape[0]), np.float32, self.ctx)
            check(lib.lumen_gemv_fused_f32(self.ctx.handle, w.ptr, 0, x.ptr, logits.ptr, w.shape[0], w.shape[1],
                                           self.norm.weight.ptr, self.norm.eps, _lib.GEMV_EPI_STORE, None))
            return logits
        x = self.norm.forward(x)
        return self.lm_head.forward(x)
