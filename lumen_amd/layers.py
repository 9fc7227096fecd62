"""Layer classes of the reference's src/layers on the GPU (inference forward only)."""
import ctypes as C
import math

import numpy as np

from ._lib import ERR_SHAPE, LumenError, check, lib
from .autograd import Tensor, default_ctx, is_no_grad
from . import ops


class Module:
    """src/module.rs:12-24 (forward / parameters / eval_mode / train_mode)."""

    def forward(self, x):
        raise NotImplementedError

    def parameters(self):
        return []

    def eval_mode(self):
        from .autograd import set_inference_mode
        set_inference_mode(True)

    def train_mode(self):
        from .autograd import set_inference_mode
        set_inference_mode(False)

    def __call__(self, *a, **k):
        return self.forward(*a, **k)


class Linear(Module):
    """src/layers/basic/linear.rs:7-50, no-bias form: weight [out, in], forward = matmul(x, W)."""

    def __init__(self, weight):
        self.weight = weight if isinstance(weight, Tensor) else Tensor.from_array_no_grad(weight)
        self.bias = None

    @staticmethod
    def new_no_bias(in_features, out_features, ctx=None):  # linear.rs:25-29 (weights start at zero here)
        return Linear(Tensor.from_array_no_grad(np.zeros((out_features, in_features), np.float32), ctx))

    def forward(self, x):  # linear.rs:33-41
        return ops.matmul(x, self.weight)

    def parameters(self):
        return [self.weight]


class RMSNorm(Module):
    """src/layers/norm/rms_norm.rs:8-62: weight [dim] (ones at construction), eps."""

    def __init__(self, dim, eps, weight=None, ctx=None):
        w = np.ones(dim, np.float32) if weight is None else np.ascontiguousarray(weight, np.float32)
        self.weight = Tensor.from_array_no_grad(w, ctx)
        self.eps = float(eps)

    def forward(self, x):
        dim = x.shape[-1]
        if dim != self.weight.shape[0]:
            raise LumenError(ERR_SHAPE, "RMSNorm: last dim %d vs weight %d" % (dim, self.weight.shape[0]))
        out = Tensor.empty(x.shape, np.float32, x.ctx)
        check(lib.lumen_rmsnorm_f32(x.ctx.handle, x.ptr, self.weight.ptr, out.ptr, x.size // dim, dim, self.eps))
        return out

    def parameters(self):
        return [self.weight]


class SiLU(Module):
    """src/layers/activation.rs:131-170 forward."""

    def forward(self, x):
        out = Tensor.empty(x.shape, np.float32, x.ctx)
        check(lib.lumen_silu_f32(x.ctx.handle, x.ptr, out.ptr, x.size))
        return out


class Embedding(Module):
    """src/layers/basic/embedding.rs:9-57: weight [vocab, dim]; indices arrive as f32 (host array)."""

    def __init__(self, weight):
        self.weight = weight if isinstance(weight, Tensor) else Tensor.from_array_no_grad(weight)
        self.vocab_size, self.embed_dim = self.weight.shape

    def forward(self, indices):
        ids = np.ascontiguousarray(indices, np.float32)
        out = Tensor.empty(ids.shape + (self.embed_dim,), np.float32, self.weight.ctx)
        check(lib.lumen_embedding_f32(self.weight.ctx.handle, self.weight.ptr, ids.ctypes.data, ids.size,
                                      self.vocab_size, self.embed_dim, out.ptr))
        return out

    def parameters(self):
        return [self.weight]


class RotaryEmbedding:
    """src/layers/attention/encoding.rs:6-231."""

    def __init__(self, dim, max_seq_len, theta, ctx=None):
        self.ctx = ctx or default_ctx()
        self.dim, self.max_seq_len, self.theta = dim, max_seq_len, theta
        h = C.c_void_p()
        check(lib.lumen_rope_create(self.ctx.handle, dim, max_seq_len, float(theta), C.byref(h)))
        self.handle = h

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            lib.lumen_rope_destroy(h)

    def tables(self):
        cos = np.empty((self.max_seq_len, self.dim), np.float32)
        sin = np.empty((self.max_seq_len, self.dim), np.float32)
        check(lib.lumen_rope_tables_download(self.handle, cos.ctypes.data, sin.ctypes.data))
        return cos, sin

    def forward(self, x, offset):  # encoding.rs:56-123, x [B,H,S,D]
        b, h, s, d = x.shape
        out = Tensor.empty(x.shape, np.float32, x.ctx)
        check(lib.lumen_rope_forward_f32(self.handle, x.ptr, out.ptr, b, h, s, d, offset))
        return out

    def rope_1token_copy(self, src, dst, pos):  # encoding.rs:173-204
        check(lib.lumen_rope_1token_copy_f32(self.handle, src.ptr, dst.ptr, src.size, pos))

    def cos_sin_row_vec(self, pos):  # encoding.rs:208-229
        if pos >= self.max_seq_len:
            from ._lib import ERR_ROPE_RANGE
            raise LumenError(ERR_ROPE_RANGE, "RoPE index out of range: pos %d >= max %d" % (pos, self.max_seq_len))
        cos, sin = self.tables()
        return cos[pos].copy(), sin[pos].copy()


class KVCacheInner:
    """src/layers/attention/self_attention.rs:24-44: k, v [B, H_kv, max_seq, D] in HBM + len."""

    def __init__(self, b, h_kv, max_seq, d, ctx=None):
        self.ctx = ctx or default_ctx()
        self.shape = (b, h_kv, max_seq, d)
        h = C.c_void_p()
        check(lib.lumen_kv_cache_create(self.ctx.handle, b, h_kv, max_seq, d, C.byref(h)))
        self.handle = h

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            lib.lumen_kv_cache_destroy(h)

    @property
    def len(self):
        n = C.c_int()
        check(lib.lumen_kv_cache_len(self.handle, C.byref(n)))
        return n.value

    @len.setter
    def len(self, n):  # a public field in the reference (self_attention.rs:28)
        check(lib.lumen_kv_cache_set_len(self.handle, int(n)))

    def reset(self):
        check(lib.lumen_kv_cache_reset(self.handle))

    def _download(self, which):
        kp, vp = C.c_void_p(), C.c_void_p()
        check(lib.lumen_kv_cache_ptrs(self.handle, C.byref(kp), C.byref(vp)))
        out = np.empty(self.shape, np.float32)
        check(lib.lumen_download(self.ctx.handle, out.ctypes.data, kp if which == "k" else vp, out.nbytes))
        return out

    @property
    def k(self):
        return self._download("k")

    @property
    def v(self):
        return self._download("v")


class SelfAttention(Module):
    """src/layers/attention/self_attention.rs:46-470, inference paths (decode S == 1, prefill S > 1)."""

    def __init__(self, embed_dim, n_head, n_kv_head, max_seq_len, rope_theta, causal, ctx=None):
        if embed_dim % n_head:  # :69-73
            raise LumenError(ERR_SHAPE, "Embed dim must be divisible by n_head")
        self.ctx = ctx or default_ctx()
        self.n_head, self.n_kv_head = n_head, n_kv_head
        self.head_dim = embed_dim // n_head
        kv_dim = n_kv_head * self.head_dim
        self.w_q = Linear.new_no_bias(embed_dim, embed_dim, self.ctx)
        self.w_k = Linear.new_no_bias(embed_dim, kv_dim, self.ctx)
        self.w_v = Linear.new_no_bias(embed_dim, kv_dim, self.ctx)
        self.w_o = Linear.new_no_bias(embed_dim, embed_dim, self.ctx)
        self.rope = RotaryEmbedding(self.head_dim, max_seq_len, rope_theta, self.ctx)
        self.scale = float(np.float32(1.0) / np.sqrt(np.float32(self.head_dim)))  # :89
        self.causal = causal
        self.max_seq = max_seq_len

    def forward(self, x, cache=None):
        """x [B, S, E]; returns (out [B, S, E], cache)."""
        if not is_no_grad():
            raise NotImplementedError("train path (self_attention.rs:429-469) is outside this build")
        b, s, _ = x.shape
        h, h_kv, d = self.n_head, self.n_kv_head, self.head_dim
        q = self.w_q.forward(x)  # :106-108
        k = self.w_k.forward(x)
        v = self.w_v.forward(x)
        if cache is None:  # :119-122
            cache = KVCacheInner(b, h_kv, self.max_seq, d, self.ctx)
        ctx_t = Tensor.empty((b, s, h, d), np.float32, x.ctx)
        if s == 1:  # :125-306
            check(lib.lumen_attn_decode_f32(cache.handle, self.rope.handle, q.ptr, k.ptr, v.ptr, ctx_t.ptr, h,
                                            self.scale, int(self.causal)))
        else:  # :308-427
            check(lib.lumen_attn_prefill_f32(cache.handle, self.rope.handle, q.ptr, k.ptr, v.ptr, ctx_t.ptr, s, h,
                                             self.scale, int(self.causal)))
        out = self.w_o.forward(ctx_t.reshape((b, s, h * d)))  # :300-303 / :421-424
        return out, cache

    def parameters(self):
        return [self.w_q.weight, self.w_k.weight, self.w_v.weight, self.w_o.weight]
