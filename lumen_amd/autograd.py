"""Tensor handle and the no_grad / inference-mode switches.

Mirrors the API shape of the reference's src/autograd.rs that the inference
path touches: Tensor (:53-64), from_array_no_grad (:162), data (:106),
data_ref-style shape access, no_grad (:47-50), is_no_grad (:43-45),
set_inference_mode (:29-31).  A Tensor here is a ref-counted f32 buffer in
HBM plus a shape; the backward machinery is out of scope.
"""
import contextlib
import ctypes as C

import numpy as np

from . import _lib
from ._lib import check, lib

_NO_GRAD_DEPTH = 0
_INFERENCE_MODE = False
_DEFAULT_CTX = None


class Context:
    """Owns a lumen_ctx (one device, one stream)."""

    def __init__(self, device=0):
        h = C.c_void_p()
        check(lib.lumen_ctx_create(device, C.byref(h)))
        self.handle = h

    @property
    def num_cus(self):
        v = C.c_int()
        check(lib.lumen_ctx_num_cus(self.handle, C.byref(v)))
        return v.value

    def synchronize(self):
        check(lib.lumen_ctx_synchronize(self.handle))

    def timer_start(self):
        check(lib.lumen_timer_start(self.handle))

    def timer_stop(self):
        ms = C.c_float()
        check(lib.lumen_timer_stop(self.handle, C.byref(ms)))
        return ms.value

    def __del__(self):
        h, self.handle = getattr(self, "handle", None), None
        if h:
            lib.lumen_ctx_destroy(h)


def default_ctx():
    global _DEFAULT_CTX
    if _DEFAULT_CTX is None:
        _DEFAULT_CTX = Context(0)
    return _DEFAULT_CTX


def set_inference_mode(on):  # autograd.rs:29-31
    global _INFERENCE_MODE
    _INFERENCE_MODE = bool(on)


def is_no_grad():  # autograd.rs:43-45
    return _NO_GRAD_DEPTH > 0 or _INFERENCE_MODE


@contextlib.contextmanager
def no_grad():  # autograd.rs:47-50 (NoGradGuard)
    global _NO_GRAD_DEPTH
    _NO_GRAD_DEPTH += 1
    try:
        yield
    finally:
        _NO_GRAD_DEPTH -= 1


class _Buffer:
    """Device allocation freed when the last Tensor viewing it goes away (the Rc of autograd.rs:64)."""

    def __init__(self, ctx, nbytes):
        self.ctx = ctx
        p = C.c_void_p()
        check(lib.lumen_malloc(ctx.handle, nbytes, C.byref(p)))
        self.ptr = p.value
        self.nbytes = nbytes

    def __del__(self):
        if getattr(self, "ptr", None) and self.ctx.handle:
            lib.lumen_free(self.ctx.handle, self.ptr)
            self.ptr = None


class Tensor:
    """f32 (or bf16-bits) array in HBM with a shape; views share the buffer."""

    def __init__(self, buf, shape, dtype=np.float32, offset=0):
        self._buf = buf
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self._offset = offset

    # -- constructors -----------------------------------------------------
    @staticmethod
    def empty(shape, dtype=np.float32, ctx=None):
        ctx = ctx or default_ctx()
        n = int(np.prod(shape)) if len(shape) else 1
        return Tensor(_Buffer(ctx, max(n, 1) * np.dtype(dtype).itemsize), shape, dtype)

    @staticmethod
    def from_array_no_grad(a, ctx=None):  # autograd.rs:162-164
        a = np.ascontiguousarray(a)
        if a.dtype not in (np.float32, np.uint16):
            a = a.astype(np.float32)
        t = Tensor.empty(a.shape, a.dtype, ctx)
        if a.size:
            check(lib.lumen_upload(t.ctx.handle, t.ptr, a.ctypes.data, a.nbytes))
        return t

    # -- access -----------------------------------------------------------
    @property
    def ctx(self):
        return self._buf.ctx

    @property
    def ptr(self):
        return self._buf.ptr + self._offset

    @property
    def size(self):
        return int(np.prod(self.shape)) if len(self.shape) else 1

    def data(self):  # autograd.rs:106-108: owned host copy
        out = np.empty(self.shape, self.dtype)
        if out.size:
            check(lib.lumen_download(self.ctx.handle, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def requires_grad(self):
        return False

    def reshape(self, shape):  # ops/shape.rs:9-49: contiguous data, metadata only
        shape = [int(s) for s in shape]
        if -1 in shape:
            known = int(np.prod([s for s in shape if s != -1]))
            shape[shape.index(-1)] = self.size // max(known, 1)
        if int(np.prod(shape)) != self.size:
            raise ValueError("Reshape failed: Total element count mismatch")
        return Tensor(self._buf, shape, self.dtype, self._offset)

    def __add__(self, other):  # ops/arithmetic.rs:48-51 (same shape)
        from . import ops
        return ops.add(self, other)

    def __mul__(self, other):  # ops/arithmetic.rs:105-108 (same shape)
        from . import ops
        return ops.mul(self, other)
