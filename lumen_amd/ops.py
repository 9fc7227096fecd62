"""Operator functions of the reference's src/ops on the GPU."""
import ctypes as C

import numpy as np

from ._lib import ERR_SHAPE, LumenError, check, lib
from .autograd import Tensor


def matmul(a, b):
    """ops::matmul::matmul (src/ops/matmul.rs:10-99): a [..., K] @ b[N, K]^T -> [..., N].

    b must be 2-D and its K must equal a's last dimension, else a SHAPE error
    (the reference panics, :24-38).  One row (M == 1) runs the GEMV, more the
    MFMA GEMM.  b may hold bf16 bits (dtype uint16).
    """
    if len(b.shape) != 2:
        raise LumenError(ERR_SHAPE, "MatMul RHS must be 2D, got %s" % (b.shape,))
    k_a = a.shape[-1]
    n, k_w = b.shape
    m = a.size // k_a if k_a else 0
    out = Tensor.empty(a.shape[:-1] + (n,), np.float32, a.ctx)
    h = a.ctx.handle
    if b.dtype == np.uint16:
        if k_a != k_w:
            raise LumenError(ERR_SHAPE, "MatMul shape mismatch: a (K=%d) vs b (K=%d)" % (k_a, k_w))
        if m == 1:
            check(lib.lumen_gemv_bf16w(h, b.ptr, a.ptr, out.ptr, n, k_a))
        else:
            check(lib.lumen_gemm_bf16w(h, a.ptr, b.ptr, out.ptr, m, n, k_a))
    else:
        check(lib.lumen_matmul_f32(h, a.ptr, b.ptr, out.ptr, m, n, k_a, k_w))
    return out


def _same_shape(a, b, what):
    if a.shape != b.shape:
        raise LumenError(ERR_SHAPE, "%s: shapes %s and %s differ (broadcasting is outside the inference path)"
                         % (what, a.shape, b.shape))


def add(a, b):  # src/ops/arithmetic.rs:48-51
    _same_shape(a, b, "add")
    out = Tensor.empty(a.shape, np.float32, a.ctx)
    check(lib.lumen_add_f32(a.ctx.handle, a.ptr, b.ptr, out.ptr, a.size))
    return out


def mul(a, b):  # src/ops/arithmetic.rs:105-108
    _same_shape(a, b, "mul")
    out = Tensor.empty(a.shape, np.float32, a.ctx)
    check(lib.lumen_mul_f32(a.ctx.handle, a.ptr, b.ptr, out.ptr, a.size))
    return out


def swiglu(gate, up):  # silu(gate) * up, src/models/llama.rs:60-63 in one pass
    _same_shape(gate, up, "swiglu")
    out = Tensor.empty(gate.shape, np.float32, gate.ctx)
    check(lib.lumen_swiglu_f32(gate.ctx.handle, gate.ptr, up.ptr, out.ptr, gate.size))
    return out


def reshape(t, shape):  # src/ops/shape.rs:9-49
    return t.reshape(shape)


def argmax(t):
    import ctypes as C
    idx = C.c_int()
    check(lib.lumen_argmax_f32(t.ctx.handle, t.ptr, t.size, C.byref(idx)))
    return idx.value


def sample_top_p(logits, temperature, top_p, repetition_penalty, recent_tokens, r):
    """sample_top_p, src/main.rs:74-137, on host logits with the uniform draw r given."""
    x = np.ascontiguousarray(logits, np.float32)
    rec = np.ascontiguousarray(recent_tokens, np.int32)
    out = C.c_int32()
    check(lib.lumen_sample_top_p_f32(x.ctypes.data, x.size, float(temperature), float(top_p), float(repetition_penalty),
                                     rec.ctypes.data, rec.size, float(r), C.byref(out)))
    return out.value


def rand01_stream(seed, n):
    """The first n draws of the seeded generator behind lumen_llama_generate_turn."""
    state = C.c_uint64(seed)
    return np.array([lib.lumen_rand01(C.byref(state)) for _ in range(n)], np.float32)
