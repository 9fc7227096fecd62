"""GPU check of lumen_attn_decode_static_f32, the decode-attention entry point that allocates nothing: its
scratch (the partial states of a sliced long cache, as tagged words, and the launch count their tags are made
of) is a fixed array in the library's device image.  It must give the same bits as lumen_attn_decode_f32 -- outputs and appended cache rows -- on calls in a
row that share the array, the later ones smaller than the first, and refuse what the array cannot hold."""
import math

import numpy as np
import pytest

from lumen_amd import _lib
from lumen_amd._lib import check, lib
from lumen_amd.autograd import Tensor
from lumen_amd.layers import KVCacheInner, RotaryEmbedding
from oracle import lumen_oracle as lo
from tests.gpu_util import dev, f32, max_rel

pytestmark = pytest.mark.gpu


def _filled_pair(rng, h_kv, d, max_seq, filled):
    """Two device caches with the same `filled` rows, and the checker's cache beside them."""
    a, b, o = (KVCacheInner(1, h_kv, max_seq, d), KVCacheInner(1, h_kv, max_seq, d), lo.KVCache(1, h_kv, max_seq, d))
    k0 = f32(rng.normal(0, 1, (1, h_kv, filled, d)))
    v0 = f32(rng.normal(0, 1, (1, h_kv, filled, d)))
    kd, vd = dev(k0), dev(v0)
    for c in (a, b):
        check(lib.lumen_kv_cache_update(c.handle, kd.ptr, vd.ptr, filled, 0))
        c.len = filled
    o.k[:, :, :filled] = k0
    o.v[:, :, :filled] = v0
    o._c.contents.len = filled
    return a, b, o


def _step(fn, cache, rope, q, k, v, h, scale):
    out = Tensor.empty((1, 1, h, q.shape[-1]))
    qd, kd, vd = dev(q), dev(k), dev(v)
    check(fn(cache.handle, rope.handle, qd.ptr, kd.ptr, vd.ptr, out.ptr, h, scale, 1))
    return out.data()


def test_static_scratch_decode_attention_matches_the_allocating_entry_point():
    rng = np.random.default_rng(77)
    # first a large call (32 heads, 16 slices, all in use), then smaller ones that find its leftovers in the array
    for h, h_kv, d, max_seq, filled in [(32, 4, 64, 4096, 3990), (4, 2, 64, 1024, 700), (2, 1, 128, 640, 300),
                                        (8, 2, 64, 2048, 40)]:
        scale = 1.0 / math.sqrt(d)
        rope = RotaryEmbedding(d, max_seq, 10000.0)
        cos, sin = lo.rope_table(d, max_seq, 10000.0)
        a, b, o = _filled_pair(rng, h_kv, d, max_seq, filled)
        for t in range(3):
            q = f32(rng.normal(0, 1, (1, h, d)))
            k = f32(rng.normal(0, 1, (1, h_kv, d)))
            v = f32(rng.normal(0, 1, (1, h_kv, d)))
            want = _step(lib.lumen_attn_decode_f32, a, rope, q, k, v, h, scale)
            got = _step(lib.lumen_attn_decode_static_f32, b, rope, q, k, v, h, scale)
            rc, ref = lo.attn_decode(o, q, k, v, cos, sin, scale)
            assert rc == lo.LO_OK and max_rel(want, ref) <= 2e-5
            assert np.array_equal(got, want), (h, d, filled, t)
            assert a.len == b.len == o.len == filled + t + 1
        n = filled + 3
        assert np.array_equal(b.k[:, :, filled:n], o.k[:, :, filled:n]) and np.array_equal(b.v[:, :, filled:n], o.v[:, :, filled:n])


def test_static_scratch_refuses_what_it_cannot_hold():
    d, max_seq = 128, 8192  # 64 slices x 130 words x 8 bytes = 66 KB per head: 256 heads do not fit 4 MiB
    rope = RotaryEmbedding(d, max_seq, 10000.0)
    c = KVCacheInner(1, 2, max_seq, d)
    q, kv = dev(np.zeros((1, 256, d), np.float32)), dev(np.zeros((1, 2, d), np.float32))
    out = Tensor.empty((1, 1, 256, d))
    rc = lib.lumen_attn_decode_static_f32(c.handle, rope.handle, q.ptr, kv.ptr, kv.ptr, out.ptr, 256, 0.1, 1)
    assert rc == _lib.ERR_UNSUPPORTED and b"static scratch" in lib.lumen_last_error()
    assert c.len == 0
    check(lib.lumen_attn_decode_f32(c.handle, rope.handle, q.ptr, kv.ptr, kv.ptr, out.ptr, 256, 0.1, 1))
    assert c.len == 1
