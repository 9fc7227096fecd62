"""GPU parity: static KV cache, decode attention and prefill attention against the CPU oracle.

Cache rows (RoPE(k), v) must be bit-exact; attention outputs within 2e-5 of max|ref| (the
online-softmax merge order differs from the reference's sequential scan).
"""
import math

import numpy as np
import pytest

from lumen_amd import _lib
from lumen_amd.kv_cache import LlamaKVCache
from lumen_amd.layers import KVCacheInner, RotaryEmbedding
from lumen_amd.models import LlamaConfig
from lumen_amd._lib import check, lib
from lumen_amd.autograd import Tensor
from oracle import lumen_oracle as lo
from tests.gpu_util import dev, f32, max_rel

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(7)
TOL = 2e-5


def gpu_decode(cache, rope, q, k, v, h, scale):
    out = Tensor.empty((q.shape[0], 1, h, q.shape[-1]))
    qd, kd, vd = dev(q), dev(k), dev(v)  # keep the device buffers alive across the call
    check(lib.lumen_attn_decode_f32(cache.handle, rope.handle, qd.ptr, kd.ptr, vd.ptr, out.ptr, h, scale, 1))
    return out.data()


def gpu_prefill(cache, rope, q, k, v, scale):
    b, s, h, d = q.shape
    out = Tensor.empty((b, s, h, d))
    qd, kd, vd = dev(q), dev(k), dev(v)
    check(lib.lumen_attn_prefill_f32(cache.handle, rope.handle, qd.ptr, kd.ptr, vd.ptr, out.ptr, s, h, scale, 1))
    return out.data()


@pytest.mark.parametrize("h,h_kv,d,max_seq,prefill,steps", [
    (32, 4, 64, 2048, 0, 40), (32, 4, 64, 2048, 300, 6), (16, 8, 128, 512, 100, 5), (32, 32, 128, 256, 61, 4),
    (8, 2, 16, 64, 0, 64), (8, 1, 32, 4096, 4000, 3), (2, 2, 64, 32, 1, 3),
    (6, 2, 64, 640, 250, 4), (28, 4, 128, 1024, 300, 3), (5, 1, 32, 64, 0, 6)])  # group sizes 3, 7, 5
def test_decode_steps_match_oracle(h, h_kv, d, max_seq, prefill, steps):
    scale = 1.0 / math.sqrt(d)
    rope = RotaryEmbedding(d, max_seq, 10000.0)
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    g, o = KVCacheInner(1, h_kv, max_seq, d), lo.KVCache(1, h_kv, max_seq, d)
    if prefill:
        q = f32(RNG.normal(0, 1, (1, prefill, h, d)))
        k = f32(RNG.normal(0, 1, (1, prefill, h_kv, d)))
        v = f32(RNG.normal(0, 1, (1, prefill, h_kv, d)))
        got = gpu_prefill(g, rope, q, k, v, scale)
        rc, ref = lo.attn_prefill(o, q, k, v, cos, sin, scale)
        assert rc == lo.LO_OK and max_rel(got, ref) <= TOL
    for t in range(steps):
        q = f32(RNG.normal(0, 1, (1, h, d)))
        k = f32(RNG.normal(0, 1, (1, h_kv, d)))
        v = f32(RNG.normal(0, 1, (1, h_kv, d)))
        got = gpu_decode(g, rope, q, k, v, h, scale)
        rc, ref = lo.attn_decode(o, q, k, v, cos, sin, scale)
        assert rc == lo.LO_OK
        assert max_rel(got, ref) <= TOL, (t, max_rel(got, ref))
        assert g.len == o.len == prefill + t + 1
    n = prefill + steps
    assert np.array_equal(g.k[:, :, :n], o.k[:, :, :n]) and np.array_equal(g.v[:, :, :n], o.v[:, :, :n])
    assert not g.k[:, :, n:].any() and not g.v[:, :, n:].any()  # untouched rows stay zero


@pytest.mark.parametrize("h,h_kv,d,max_seq,filled,steps", [
    (32, 4, 64, 4096, 3990, 3),     # the long-context benchmark shape: 16 slices, heads of a slice grouped per XCD
    (16, 8, 128, 2048, 1500, 3),    # head_dim 128, n_rep 2: 12 of 16 slices in use
    (32, 32, 128, 1024, 700, 2),    # one query head per KV head
    (8, 2, 16, 4096, 3000, 2),      # head_dim 16: 1024 rows per slice, 4 slices (the ungrouped placement)
    (4, 1, 64, 640, 520, 3),        # 3 of 4 slices in use
    (2, 1, 128, 16384, 9000, 2),    # longer than 64 slices of one trip: two trips per slice
    (8, 1, 32, 40000, 36000, 2),    # 64 slices of 576 rows; n_rep 8
    (12, 4, 64, 4096, 2500, 2),     # groups of three query heads, 10 of 16 slices
    (14, 2, 128, 1024, 900, 2),     # groups of seven
], ids=["d64-nrep8-4096", "d128-nrep2", "d128-mha", "d16", "d64-nrep4-short-tail", "d128-two-trips", "d32-64-slices",
        "d64-nrep3", "d128-nrep7"])
def test_decode_over_a_long_cache_filled_directly(h, h_kv, d, max_seq, filled, steps):
    """Decode attention over caches of thousands of rows: the rows are written straight into both caches
    (lumen_kv_cache_update + lumen_kv_cache_set_len here, the arrays there), so no quadratic prompt pass is needed."""
    scale = 1.0 / math.sqrt(d)
    rope = RotaryEmbedding(d, max_seq, 10000.0)
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    g, o = KVCacheInner(1, h_kv, max_seq, d), lo.KVCache(1, h_kv, max_seq, d)
    k0 = f32(RNG.normal(0, 1, (1, h_kv, filled, d)))
    v0 = f32(RNG.normal(0, 1, (1, h_kv, filled, d)))
    kd, vd = dev(k0), dev(v0)
    check(lib.lumen_kv_cache_update(g.handle, kd.ptr, vd.ptr, filled, 0))
    g.len = filled
    o.k[:, :, :filled] = k0
    o.v[:, :, :filled] = v0
    o._c.contents.len = filled
    for t in range(steps):
        q = f32(RNG.normal(0, 1, (1, h, d)))
        k = f32(RNG.normal(0, 1, (1, h_kv, d)))
        v = f32(RNG.normal(0, 1, (1, h_kv, d)))
        got = gpu_decode(g, rope, q, k, v, h, scale)
        rc, ref = lo.attn_decode(o, q, k, v, cos, sin, scale)
        assert rc == lo.LO_OK
        assert max_rel(got, ref) <= TOL, (t, max_rel(got, ref))
        assert g.len == o.len == filled + t + 1
    n = filled + steps
    assert np.array_equal(g.k[:, :, filled:n], o.k[:, :, filled:n]) and np.array_equal(g.v[:, :, filled:n], o.v[:, :, filled:n])
    with pytest.raises(_lib.LumenError) as e:
        g.len = max_seq + 1
    assert e.value.status == _lib.ERR_KV_OVERFLOW


@pytest.mark.parametrize("b,h,h_kv,d,max_seq,prefill,steps", [
    (2, 8, 2, 64, 128, 20, 4),       # short form
    (3, 4, 4, 128, 640, 300, 3),     # long form (3 slices), one head per KV head
    (2, 16, 2, 64, 1024, 200, 2),    # prompt pass on the matrix cores, then the short form
])
def test_batch_of_sequences(b, h, h_kv, d, max_seq, prefill, steps):
    """The operator entry points take a batch (KVCacheInner::new(b, ...), self_attention.rs:33); every sequence of
    the batch is at the same position."""
    scale = 1.0 / math.sqrt(d)
    rope = RotaryEmbedding(d, max_seq, 10000.0)
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    g, o = KVCacheInner(b, h_kv, max_seq, d), lo.KVCache(b, h_kv, max_seq, d)
    q = f32(RNG.normal(0, 1, (b, prefill, h, d)))
    k = f32(RNG.normal(0, 1, (b, prefill, h_kv, d)))
    v = f32(RNG.normal(0, 1, (b, prefill, h_kv, d)))
    got = gpu_prefill(g, rope, q, k, v, scale)
    rc, ref = lo.attn_prefill(o, q, k, v, cos, sin, scale)
    assert rc == lo.LO_OK and max_rel(got, ref) <= TOL
    for t in range(steps):
        q = f32(RNG.normal(0, 1, (b, h, d)))
        k = f32(RNG.normal(0, 1, (b, h_kv, d)))
        v = f32(RNG.normal(0, 1, (b, h_kv, d)))
        got = gpu_decode(g, rope, q, k, v, h, scale)
        rc, ref = lo.attn_decode(o, q, k, v, cos, sin, scale)
        assert rc == lo.LO_OK and max_rel(got, ref) <= TOL, t
    n = prefill + steps
    assert g.len == o.len == n
    assert np.array_equal(g.k[:, :, :n], o.k[:, :, :n]) and np.array_equal(g.v[:, :, :n], o.v[:, :, :n])


def test_decode_degenerate_and_gqa_mapping():
    h, h_kv, d, max_seq = 8, 2, 64, 128
    rope = RotaryEmbedding(d, max_seq, 10000.0)
    g = KVCacheInner(1, h_kv, max_seq, d)
    q = f32(RNG.normal(0, 1, (1, h, d)))
    k = f32(RNG.normal(0, 1, (1, h_kv, d)))
    v = f32(RNG.normal(0, 1, (1, h_kv, d)))
    out = gpu_decode(g, rope, q, k, v, h, 0.125)
    for hq in range(h):  # L = 1: out = v of the head's KV group
        assert np.array_equal(out[0, 0, hq], v[0, hq // 4])
    g.reset()
    vs = []
    for t in range(70):  # zero queries: uniform weights -> mean of V per KV group
        v = f32(np.stack([np.full(d, 10.0 * (grp + 1) + t) for grp in range(h_kv)])[None])
        vs.append(v[0])
        out = gpu_decode(g, rope, np.zeros((1, h, d), np.float32), f32(RNG.normal(0, 1, (1, h_kv, d))), v, h, 0.125)
    mean = np.mean(vs, 0)
    for hq in range(h):
        assert np.allclose(out[0, 0, hq], mean[hq // 4], rtol=1e-5)


def test_cache_state_machine_overflow_and_reset():
    h, h_kv, d, max_seq = 2, 1, 16, 6
    rope = RotaryEmbedding(d, max_seq, 10000.0)
    g = KVCacheInner(1, h_kv, max_seq, d)
    assert g.len == 0 and not g.k.any() and not g.v.any()
    r = lambda *s: f32(RNG.normal(0, 1, s))
    gpu_prefill(g, rope, r(1, 4, h, d), r(1, 4, h_kv, d), r(1, 4, h_kv, d), 0.25)
    assert g.len == 4
    gpu_decode(g, rope, r(1, h, d), r(1, h_kv, d), r(1, h_kv, d), h, 0.25)
    assert g.len == 5
    with pytest.raises(_lib.LumenError) as e:
        gpu_prefill(g, rope, r(1, 2, h, d), r(1, 2, h_kv, d), r(1, 2, h_kv, d), 0.25)
    assert e.value.status == _lib.ERR_ROPE_RANGE and g.len == 5
    gpu_decode(g, rope, r(1, h, d), r(1, h_kv, d), r(1, h_kv, d), h, 0.25)
    with pytest.raises(_lib.LumenError) as e:
        gpu_decode(g, rope, r(1, h, d), r(1, h_kv, d), r(1, h_kv, d), h, 0.25)
    assert e.value.status == _lib.ERR_KV_OVERFLOW and g.len == 6
    stale = g.k
    g.reset()
    assert g.len == 0 and np.array_equal(g.k, stale)
    q, k, v = r(1, h, d), r(1, h_kv, d), r(1, h_kv, d)
    a = gpu_decode(g, rope, q, k, v, h, 0.25)
    b = gpu_decode(KVCacheInner(1, h_kv, max_seq, d), rope, q, k, v, h, 0.25)
    assert np.array_equal(a, b)  # stale rows beyond len are never read


# prompts of 192 positions and more with head_dim 64 / 128 take the matrix-core kernel (n_rep 8, 2, 1, 4 here;
# lengths that are no multiple of the tile sizes, with and without rows already in the cache)
@pytest.mark.parametrize("h,h_kv,d,s,past", [(32, 4, 64, 128, 0), (16, 8, 128, 50, 17), (4, 4, 32, 3, 9), (8, 2, 16, 33, 31),
                                             (16, 2, 64, 331, 0), (8, 4, 128, 200, 45), (4, 4, 64, 193, 230),
                                             (8, 2, 64, 257, 63),
                                             (6, 2, 64, 40, 11), (12, 4, 64, 300, 21), (14, 2, 128, 210, 0),  # groups of 3, 3, 7
                                             (5, 1, 32, 70, 0)])
def test_prefill_with_and_without_past(h, h_kv, d, s, past):
    max_seq = past + s + 3
    scale = 1.0 / math.sqrt(d)
    rope = RotaryEmbedding(d, max_seq, 10000.0)
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    g, o = KVCacheInner(1, h_kv, max_seq, d), lo.KVCache(1, h_kv, max_seq, d)
    for n in ([past, s] if past else [s]):
        q = f32(RNG.normal(0, 1, (1, n, h, d)))
        k = f32(RNG.normal(0, 1, (1, n, h_kv, d)))
        v = f32(RNG.normal(0, 1, (1, n, h_kv, d)))
        got = gpu_prefill(g, rope, q, k, v, scale)
        rc, ref = lo.attn_prefill(o, q, k, v, cos, sin, scale)
        assert rc == lo.LO_OK and max_rel(got, ref) <= TOL
    assert g.len == o.len == past + s
    assert np.array_equal(g.k, o.k) and np.array_equal(g.v, o.v)


def test_legacy_llama_kv_cache_update_and_view():
    cfg = LlamaConfig(hidden_size=64, num_attention_heads=4, num_key_value_heads=2, max_seq_len=10)
    c = LlamaKVCache(cfg)
    k = f32(RNG.normal(0, 1, (1, 2, 3, 16)))
    v = f32(RNG.normal(0, 1, (1, 2, 3, 16)))
    c.update(dev(k), dev(v), 4)
    assert np.array_equal(c.k_cache[:, :, 4:7], k) and np.array_equal(c.v_cache[:, :, 4:7], v)
    assert not c.k_cache[:, :, :4].any() and not c.k_cache[:, :, 7:].any()
    kv, vv = c.get_view(6)
    assert kv.shape == (1, 2, 6, 16)
    assert np.array_equal(kv.data(), c.k_cache[:, :, :6]) and np.array_equal(vv.data(), c.v_cache[:, :, :6])
    with pytest.raises(_lib.LumenError) as e:
        c.update(dev(k), dev(v), 8)  # kv_cache.rs:33-36
    assert e.value.status == _lib.ERR_KV_OVERFLOW


@pytest.mark.parametrize("h,h_kv,d,hidden,max_seq,prefill,steps,bf16", [
    (32, 4, 64, 2048, 2048, 0, 6, False), (8, 2, 64, 512, 700, 509, 6, False), (16, 8, 128, 1024, 512, 100, 4, False),
    (4, 4, 32, 128, 64, 3, 4, False), (16, 2, 64, 1024, 4096, 4000, 3, True)])
def test_fused_qkv_rope_append_then_prerotated_attention_equals_the_unfused_step(h, h_kv, d, hidden, max_seq, prefill,
                                                                                 steps, bf16):
    """lumen_qkv_rope_append_f32 + lumen_attn_decode_prerotated_f32 against the checker's leaves: RMSNorm, the
    three projections, then the decode attention core (which rotates, appends and attends).  The new cache row
    and the output agree to the rounding of the projection sums; the length advances in the second call only;
    overflow and RoPE range are refused before anything is written."""
    rng = np.random.default_rng(h * 131 + d + prefill)
    scale = 1.0 / math.sqrt(d)
    rope = RotaryEmbedding(d, max_seq, 10000.0)
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    g, o = KVCacheInner(1, h_kv, max_seq, d), lo.KVCache(1, h_kv, max_seq, d)
    if prefill:
        q = f32(rng.normal(0, 1, (1, prefill, h, d)))
        k = f32(rng.normal(0, 1, (1, prefill, h_kv, d)))
        v = f32(rng.normal(0, 1, (1, prefill, h_kv, d)))
        gpu_prefill(g, rope, q, k, v, scale)
        lo.attn_prefill(o, q, k, v, cos, sin, scale)
    W = f32(rng.normal(0, 0.05, ((h + 2 * h_kv) * d, hidden)))
    Wh = lo.f32_to_bf16(W) if bf16 else W
    Wref = lo.bf16_to_f32(Wh) if bf16 else W
    gains = f32(rng.normal(1, 0.2, hidden))
    Wd, gd = dev(Wh), dev(gains)
    tol = 3e-5
    for t in range(steps):
        x = f32(rng.normal(0, 1, hidden))
        xd = dev(x)
        q_rot, out = Tensor.empty((h * d,)), Tensor.empty((h * d,))
        check(lib.lumen_qkv_rope_append_f32(g.handle, rope.handle, Wd.ptr, int(bf16), xd.ptr, hidden, gd.ptr, 1e-5, q_rot.ptr, h))
        assert g.len == prefill + t  # not advanced yet
        check(lib.lumen_attn_decode_prerotated_f32(g.handle, q_rot.ptr, out.ptr, h, scale))
        assert g.len == prefill + t + 1
        xn = lo.rmsnorm(x[None], gains, 1e-5)[0]
        qkv = lo.gemv(Wref, xn)
        q3 = qkv[:h * d].reshape(1, h, d)
        k3 = qkv[h * d:(h + h_kv) * d].reshape(1, h_kv, d)
        v3 = qkv[(h + h_kv) * d:].reshape(1, h_kv, d)
        rc, ref = lo.attn_decode(o, f32(q3), f32(k3), f32(v3), cos, sin, scale)
        assert rc == lo.LO_OK
        assert max_rel(out.data(), ref.reshape(-1)) <= tol, t
        n = o.len
        assert max_rel(g.k[:, :, n - 1], o.k[:, :, n - 1]) <= tol and max_rel(g.v[:, :, n - 1], o.v[:, :, n - 1]) <= tol
        q_ref = np.stack([lo.rope_1token_copy(f32(q3[0, i]), cos, sin, n - 1)[1] for i in range(h)])
        assert max_rel(q_rot.data().reshape(h, d), q_ref) <= tol
    if prefill + steps < max_seq and max_seq <= 64:
        g.len = max_seq  # full cache: self_attention.rs:144-149
        with pytest.raises(_lib.LumenError) as e:
            check(lib.lumen_qkv_rope_append_f32(g.handle, rope.handle, Wd.ptr, int(bf16), xd.ptr, hidden, gd.ptr, 1e-5, q_rot.ptr, h))
        assert e.value.status == _lib.ERR_KV_OVERFLOW
        with pytest.raises(_lib.LumenError) as e:
            check(lib.lumen_attn_decode_prerotated_f32(g.handle, q_rot.ptr, out.ptr, h, scale))
        assert e.value.status == _lib.ERR_KV_OVERFLOW
