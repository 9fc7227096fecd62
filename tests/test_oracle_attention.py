"""Pins the oracle's KV cache, decode attention and prefill attention.

Checks are independent of the restated formulas: fp64 two-pass softmax,
degenerate inputs with known answers, the GQA head mapping made visible by
per-group-distinct values, cross-path consistency (decode == last row of
prefill, chunked prefill == single prefill) and torch's
scaled_dot_product_attention.
"""
import math

import numpy as np
import pytest
import torch

from oracle import lumen_oracle as lo

RNG = np.random.default_rng(4321)


def f32(a):
    return np.ascontiguousarray(a, np.float32)


def rope64(x, pos, d, theta=10000.0):
    """fp64 half-split rotation of the last axis at absolute position pos."""
    half = d // 2
    ang = pos * theta ** (-2.0 * np.arange(half) / d)
    c, s = np.cos(ang), np.sin(ang)
    x = x.astype(np.float64)
    return np.concatenate([x[..., :half] * c - x[..., half:] * s, x[..., half:] * c + x[..., :half] * s], -1)


def fill_cache_by_decode(cache, steps, h, h_kv, d, cos, sin, scale):
    outs, qs, ks, vs = [], [], [], []
    for _ in range(steps):
        q = f32(RNG.normal(0, 1, (1, h, d)))
        k = f32(RNG.normal(0, 1, (1, h_kv, d)))
        v = f32(RNG.normal(0, 1, (1, h_kv, d)))
        rc, out = lo.attn_decode(cache, q, k, v, cos, sin, scale)
        assert rc == lo.LO_OK
        outs.append(out); qs.append(q); ks.append(k); vs.append(v)
    return outs, qs, ks, vs


@pytest.mark.parametrize("h,h_kv,d,steps", [(4, 2, 16, 9), (8, 2, 64, 33), (2, 2, 128, 5), (32, 4, 64, 20)])
def test_decode_matches_fp64_two_pass_softmax(h, h_kv, d, steps):
    max_seq = 64
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    scale = 1.0 / math.sqrt(d)
    cache = lo.KVCache(1, h_kv, max_seq, d)
    outs, qs, ks, vs = fill_cache_by_decode(cache, steps, h, h_kv, d, cos, sin, scale)
    assert cache.len == steps
    n_rep = h // h_kv
    K = np.stack([rope64(ks[t][0], t, d) for t in range(steps)], 1)      # [h_kv, L, d]
    V = np.stack([vs[t][0].astype(np.float64) for t in range(steps)], 1)
    # cache rows hold RoPE(k) at their absolute position and raw v
    assert np.allclose(cache.k[0, :, :steps], K, rtol=1e-5, atol=1e-5)
    assert np.array_equal(cache.v[0, :, :steps], V.astype(np.float32))
    for t in (0, steps // 2, steps - 1):
        qr = rope64(qs[t][0], t, d)
        for hq in range(h):
            hk = hq // n_rep
            sc = (K[hk, :t + 1] @ qr[hq]) * scale
            p = np.exp(sc - sc.max())
            ref = (p / p.sum()) @ V[hk, :t + 1]
            assert np.allclose(outs[t][0, 0, hq], ref, rtol=2e-5, atol=2e-6)


def test_decode_degenerate_cases():
    h, h_kv, d, max_seq = 4, 2, 8, 16
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    cache = lo.KVCache(1, h_kv, max_seq, d)
    q = f32(RNG.normal(0, 1, (1, h, d)))
    k = f32(RNG.normal(0, 1, (1, h_kv, d)))
    v = f32(RNG.normal(0, 1, (1, h_kv, d)))
    rc, out = lo.attn_decode(cache, q, k, v, cos, sin, 0.3)
    # L = 1: softmax over one key -> out = v / (1 + 1e-9) = v in f32, for every q head of the group
    for hq in range(h):
        assert np.array_equal(out[0, 0, hq], v[0, hq // 2])
    # zero queries -> uniform weights -> mean of V; distinct V per kv head exposes the GQA mapping
    cache.reset()
    vs = []
    for t in range(5):
        v = f32(np.stack([np.full(d, 10.0 * (g + 1) + t) for g in range(h_kv)])[None])
        vs.append(v)
        rc, out = lo.attn_decode(cache, f32(np.zeros((1, h, d))), f32(RNG.normal(0, 1, (1, h_kv, d))), v, cos, sin, 0.3)
    mean = np.mean([x[0] for x in vs], 0)
    for hq in range(h):
        assert np.allclose(out[0, 0, hq], mean[hq // 2], rtol=1e-6)
    assert not np.allclose(out[0, 0, 0], out[0, 0, 2])


def test_kv_cache_state_machine_and_overflow():
    h, h_kv, d, max_seq = 2, 1, 8, 6
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    cache = lo.KVCache(1, h_kv, max_seq, d)
    assert cache.len == 0 and not cache.k.any() and not cache.v.any()           # zero-init (:33-39)
    q = f32(RNG.normal(0, 1, (1, 4, h, d)))
    k = f32(RNG.normal(0, 1, (1, 4, h_kv, d)))
    v = f32(RNG.normal(0, 1, (1, 4, h_kv, d)))
    assert lo.attn_prefill(cache, q, k, v, cos, sin, 0.3)[0] == lo.LO_OK
    assert cache.len == 4
    one = lambda n: f32(RNG.normal(0, 1, (1, n, d)))
    assert lo.attn_decode(cache, one(h), one(h_kv), one(h_kv), cos, sin, 0.3)[0] == lo.LO_OK
    assert cache.len == 5
    assert lo.attn_prefill(cache, q[:, :2].copy(), k[:, :2].copy(), v[:, :2].copy(), cos, sin, 0.3)[0] == lo.LO_ERR_ROPE_RANGE
    assert cache.len == 5                                                        # failed call leaves len alone
    assert lo.attn_decode(cache, one(h), one(h_kv), one(h_kv), cos, sin, 0.3)[0] == lo.LO_OK
    assert cache.len == 6
    assert lo.attn_decode(cache, one(h), one(h_kv), one(h_kv), cos, sin, 0.3)[0] == lo.LO_ERR_KV_OVERFLOW  # :144-149
    stale = cache.k.copy()
    cache.reset()                                                                # :41-43 len = 0, data kept
    assert cache.len == 0 and np.array_equal(cache.k, stale)
    # stale rows beyond len are never read: same answer as from a fresh cache
    qn, kn, vn = one(h), one(h_kv), one(h_kv)
    _, a = lo.attn_decode(cache, qn, kn, vn, cos, sin, 0.3)
    fresh = lo.KVCache(1, h_kv, max_seq, d)
    _, b = lo.attn_decode(fresh, qn, kn, vn, cos, sin, 0.3)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("h,h_kv,d,s,past", [(4, 2, 16, 7, 0), (8, 2, 64, 12, 5), (4, 4, 32, 3, 9)])
def test_prefill_matches_fp64_causal_softmax_and_sdpa(h, h_kv, d, s, past):
    max_seq = 32
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    scale = 1.0 / math.sqrt(d)
    cache = lo.KVCache(1, h_kv, max_seq, d)
    n_rep = h // h_kv
    allq = f32(RNG.normal(0, 1, (1, past + s, h, d)))
    allk = f32(RNG.normal(0, 1, (1, past + s, h_kv, d)))
    allv = f32(RNG.normal(0, 1, (1, past + s, h_kv, d)))
    if past:
        rc, _ = lo.attn_prefill(cache, f32(allq[:, :past]), f32(allk[:, :past]), f32(allv[:, :past]), cos, sin, scale)
        assert rc == lo.LO_OK
    rc, out = lo.attn_prefill(cache, f32(allq[:, past:]), f32(allk[:, past:]), f32(allv[:, past:]), cos, sin, scale)
    assert rc == lo.LO_OK and cache.len == past + s
    L = past + s
    Q = np.stack([rope64(allq[0, t], t, d) for t in range(L)], 0)            # [L, h, d]
    K = np.stack([rope64(allk[0, t], t, d) for t in range(L)], 0)
    V = allv[0].astype(np.float64)
    for i in range(s):
        qa = past + i
        for hq in range(h):
            hk = hq // n_rep
            sc = (K[:qa + 1, hk] @ Q[qa, hq]) * scale
            p = np.exp(sc - sc.max())
            ref = (p / p.sum()) @ V[:qa + 1, hk]
            assert np.allclose(out[0, i, hq], ref, rtol=2e-5, atol=2e-6)
    # torch SDPA with an explicit causal mask shifted by past, GQA by repeat_interleave
    qt = torch.from_numpy(Q[past:]).permute(1, 0, 2)[None]
    kt = torch.from_numpy(K).permute(1, 0, 2)[None].repeat_interleave(n_rep, 1)
    vt = torch.from_numpy(V).permute(1, 0, 2)[None].repeat_interleave(n_rep, 1)
    mask = torch.arange(L)[None, :] <= (past + torch.arange(s))[:, None]
    ref = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=mask, scale=scale)
    assert np.allclose(out[0], ref[0].permute(1, 0, 2).numpy(), rtol=2e-5, atol=2e-6)


def test_chunked_prefill_equals_single_prefill_and_decode_equals_last_row():
    h, h_kv, d, max_seq, L = 8, 2, 32, 40, 21
    cos, sin = lo.rope_table(d, max_seq, 10000.0)
    scale = 1.0 / math.sqrt(d)
    q = f32(RNG.normal(0, 1, (1, L, h, d)))
    k = f32(RNG.normal(0, 1, (1, L, h_kv, d)))
    v = f32(RNG.normal(0, 1, (1, L, h_kv, d)))
    c1 = lo.KVCache(1, h_kv, max_seq, d)
    _, full = lo.attn_prefill(c1, q, k, v, cos, sin, scale)
    c2 = lo.KVCache(1, h_kv, max_seq, d)
    _, a = lo.attn_prefill(c2, f32(q[:, :8]), f32(k[:, :8]), f32(v[:, :8]), cos, sin, scale)
    _, b = lo.attn_prefill(c2, f32(q[:, 8:L - 1]), f32(k[:, 8:L - 1]), f32(v[:, 8:L - 1]), cos, sin, scale)
    _, last = lo.attn_decode(c2, f32(q[:, L - 1]), f32(k[:, L - 1]), f32(v[:, L - 1]), cos, sin, scale)
    assert np.array_equal(c1.k, c2.k) and np.array_equal(c1.v, c2.v) and c2.len == L
    assert np.allclose(np.concatenate([a, b], 1), full[:, :L - 1], rtol=1e-5, atol=1e-6)
    assert np.allclose(last[:, 0], full[:, L - 1], rtol=1e-5, atol=1e-6)
