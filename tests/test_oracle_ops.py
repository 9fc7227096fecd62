"""Pins the CPU oracle's elementwise / GEMV / norm / RoPE restatements.

The reference ships no tests or golden vectors, so each function is held to
evidence that does not repeat its own formula: fp64 shadows with a derived
error bound, known-answer inputs, brute force in pure Python on tiny shapes,
algebraic invariants and torch's own implementations of the textbook routine.
A dropped term, a wrong sign or index, or a transposed operand fails at least
one check per function.
"""
import math

import numpy as np
import pytest
import torch

from oracle import lumen_oracle as lo

RNG = np.random.default_rng(1234)


def f32(a):
    return np.ascontiguousarray(a, np.float32)


# ----------------------------------------------------------------------- GEMV
@pytest.mark.parametrize("N,K", [(1, 1), (3, 5), (17, 64), (256, 2048), (33, 1000)])
def test_gemv_fp64_shadow_bound(N, K):
    W = f32(RNG.normal(0, 0.02, (N, K)))
    x = f32(RNG.normal(0, 1, K))
    y = lo.gemv(W, x)
    ref = W.astype(np.float64) @ x.astype(np.float64)
    # sequential f32 summation: |err| <= K * 2^-24 * sum|w_i x_i| (first order)
    bound = K * 2.0 ** -24 * (np.abs(W.astype(np.float64)) @ np.abs(x.astype(np.float64))) + 1e-30
    assert np.all(np.abs(y - ref) <= bound)


def test_gemv_sequential_order_is_bit_exact_to_python_loop():
    # brute force: the exact f32 sequence sum = fl(sum + fl(w*x)), k ascending
    N, K = 4, 37
    W = f32(RNG.normal(0, 1, (N, K)))
    x = f32(RNG.normal(0, 1, K))
    y = lo.gemv(W, x)
    for n in range(N):
        s = np.float32(0.0)
        for k in range(K):
            s = np.float32(s + np.float32(W[n, k] * x[k]))
        assert y[n] == s


def test_gemv_known_answers():
    K = 48
    x = f32(RNG.normal(0, 1, K))
    assert np.array_equal(lo.gemv(f32(np.eye(K)), x), x)                      # W = I
    ones = lo.gemv(f32(np.ones((3, K))), x)
    assert np.allclose(ones, x.astype(np.float64).sum(), rtol=1e-5)            # W = ones -> sum x
    W = f32(RNG.normal(0, 1, (7, K)))
    e = np.zeros(K, np.float32)
    e[11] = 1.0
    assert np.array_equal(lo.gemv(W, e), W[:, 11])                            # one-hot picks a column
    # layout is [N, K] (out, in): a transposed read would fail on a non-square W
    Wn = f32(np.arange(6).reshape(2, 3))
    assert np.array_equal(lo.gemv(Wn, f32([1, 10, 100])), f32([210, 543]))


def test_matmul_dispatch_and_shape_errors():
    W = f32(RNG.normal(0, 1, (5, 8)))
    a1 = f32(RNG.normal(0, 1, (1, 1, 8)))
    rc, out = lo.matmul(a1, W)
    assert rc == lo.LO_OK and out.shape == (1, 1, 5)
    assert np.array_equal(out.reshape(-1), lo.gemv(W, a1.reshape(-1)))       # M == 1 -> GEMV path
    a3 = f32(RNG.normal(0, 1, (1, 3, 8)))
    rc, out = lo.matmul(a3, W)
    assert rc == lo.LO_OK and out.shape == (1, 3, 5)
    assert np.allclose(out[0], a3[0].astype(np.float64) @ W.T.astype(np.float64), rtol=1e-5, atol=1e-6)
    rc, _ = lo.matmul(f32(np.zeros((1, 7))), W)                                # K mismatch (matmul.rs:33-38)
    assert rc == lo.LO_ERR_SHAPE
    rc, _ = lo.matmul(a1, f32(np.zeros((2, 2, 2))))                            # RHS not 2-D (matmul.rs:24-26)
    assert rc == lo.LO_ERR_SHAPE


@pytest.mark.parametrize("M,N,K", [(2, 3, 5), (7, 33, 130), (16, 64, 256)])
def test_gemm_rows_equal_gemv_within_tolerance(M, N, K):
    A = f32(RNG.normal(0, 1, (M, K)))
    W = f32(RNG.normal(0, 0.02, (N, K)))
    Cm = lo.gemm(A, W)
    ref = A.astype(np.float64) @ W.T.astype(np.float64)
    scale = np.abs(ref).max()
    assert np.abs(Cm - ref).max() <= 1e-6 * scale * math.sqrt(K)
    for m in range(M):
        assert np.abs(Cm[m] - lo.gemv(W, A[m])).max() <= 1e-5 * scale


# -------------------------------------------------------------------- RMSNorm
@pytest.mark.parametrize("rows,dim,eps", [(1, 8, 1e-5), (3, 2048, 1e-5), (5, 128, 1e-6)])
def test_rmsnorm_closed_form_and_torch(rows, dim, eps):
    x = f32(RNG.normal(0, 2, (rows, dim)))
    w = f32(RNG.normal(1, 0.2, dim))
    out = lo.rmsnorm(x, w, eps)
    x64 = x.astype(np.float64)
    ref = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + eps) * w
    assert np.allclose(out, ref, rtol=2e-6, atol=1e-7)
    t = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (dim,), torch.from_numpy(w).double(), eps)
    assert np.allclose(out, t.numpy(), rtol=2e-6, atol=1e-7)
    # invariant: mean((out/w)^2) = 1 / (1 + eps/ms)
    ms = (x64 ** 2).mean(-1)
    assert np.allclose(((out / w).astype(np.float64) ** 2).mean(-1), 1.0 / (1.0 + eps / ms), rtol=1e-5)


def test_rmsnorm_scale_invariance_and_gain_is_applied():
    x = f32(RNG.normal(0, 1, (2, 64)))
    w = f32(np.linspace(0.5, 2.0, 64))
    a = lo.rmsnorm(x, w, 0.0)
    b = lo.rmsnorm(f32(x * 8.0), w, 0.0)
    assert np.allclose(a, b, rtol=1e-6)
    unit = lo.rmsnorm(x, f32(np.ones(64)), 0.0)
    assert np.allclose(a, unit * w, rtol=1e-6)


# ----------------------------------------------------------------------- RoPE
@pytest.mark.parametrize("dim,max_seq,theta", [(64, 2048, 10000.0), (128, 512, 1.0e6), (8, 16, 10000.0)])
def test_rope_table_closed_form(dim, max_seq, theta):
    cos, sin = lo.rope_table(dim, max_seq, theta)
    half = dim // 2
    assert np.array_equal(cos[:, :half], cos[:, half:]) and np.array_equal(sin[:, :half], sin[:, half:])
    j = np.arange(half, dtype=np.float64)
    pos = np.arange(max_seq, dtype=np.float64)[:, None]
    ang = pos * theta ** (-2.0 * j / dim)
    # f32 freq and f32 product: angle error <= pos * 2^-23 relative-ish; allow that
    tol = 3e-7 * (1.0 + np.abs(ang))
    assert np.all(np.abs(cos[:, :half] - np.cos(ang)) <= tol + 1e-6)
    assert np.all(np.abs(sin[:, :half] - np.sin(ang)) <= tol + 1e-6)
    assert np.array_equal(cos[0], np.ones(dim, np.float32)) and np.array_equal(sin[0], np.zeros(dim, np.float32))


def _hf_rotate_half(x):
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def test_rope_forward_matches_hf_rotate_half_and_invariants():
    b, h, s, d, off = 1, 3, 5, 16, 7
    cos, sin = lo.rope_table(d, 64, 10000.0)
    x = f32(RNG.normal(0, 1, (b, h, s, d)))
    rc, out = lo.rope_forward(x, cos, sin, off)
    assert rc == lo.LO_OK
    xt = torch.from_numpy(x).double()
    c = torch.from_numpy(cos[off:off + s]).double()
    sn = torch.from_numpy(sin[off:off + s]).double()
    ref = xt * c + _hf_rotate_half(xt) * sn                                     # HF apply_rotary_pos_emb
    assert np.allclose(out, ref.numpy(), rtol=1e-6, atol=1e-6)
    # rotation preserves the norm of every (j, j+d/2) pair
    half = d // 2
    assert np.allclose(out[..., :half] ** 2 + out[..., half:] ** 2,
                       x[..., :half] ** 2 + x[..., half:] ** 2, rtol=1e-5)
    # position 0 is the identity
    rc, out0 = lo.rope_forward(f32(x[:, :, :1]), cos, sin, 0)
    assert np.array_equal(out0, x[:, :, :1])
    # 1-token helper equals the tensor form at the same absolute position
    rc, one = lo.rope_1token_copy(f32(x[0, 1, 2]), cos, sin, off + 2)
    assert rc == lo.LO_OK and np.array_equal(one, out[0, 1, 2])


def test_rope_relative_position_property():
    d = 32
    cos, sin = lo.rope_table(d, 256, 10000.0)
    q = f32(RNG.normal(0, 1, d))
    k = f32(RNG.normal(0, 1, d))

    def dot(p, s_):
        _, qr = lo.rope_1token_copy(q, cos, sin, p)
        _, kr = lo.rope_1token_copy(k, cos, sin, s_)
        return float(qr.astype(np.float64) @ kr.astype(np.float64))

    assert abs(dot(10, 3) - dot(107, 100)) < 2e-4
    assert abs(dot(50, 50) - float(q.astype(np.float64) @ k.astype(np.float64))) < 1e-4
    assert abs(dot(10, 3) - dot(3, 10)) > 1e-3                                  # sign of the angle matters


def test_rope_range_errors():
    cos, sin = lo.rope_table(8, 16, 10000.0)
    x = f32(np.zeros((1, 1, 4, 8)))
    assert lo.rope_forward(x, cos, sin, 12)[0] == lo.LO_OK                      # 12 + 4 == max
    assert lo.rope_forward(x, cos, sin, 13)[0] == lo.LO_ERR_ROPE_RANGE          # encoding.rs:62-68
    assert lo.rope_1token_copy(x[0, 0, 0], cos, sin, 16)[0] == lo.LO_ERR_ROPE_RANGE  # encoding.rs:176-181
    assert lo.rope_1token_copy(x[0, 0, 0], cos, sin, 15)[0] == lo.LO_OK


# ------------------------------------------------------- SiLU / add / mul / misc
def test_silu_add_mul_closed_forms():
    x = f32(np.concatenate([RNG.normal(0, 3, 1000), [0.0, -100.0, 100.0, -20.0, 20.0]]))
    s = lo.silu(x)
    ref = torch.nn.functional.silu(torch.from_numpy(x).double()).numpy()
    assert np.allclose(s, ref, rtol=2e-6, atol=1e-30)
    assert s[1000] == 0.0 and s[1001] == 0.0 and s[1002] == 100.0
    a = f32(RNG.normal(0, 1, 100))
    b = f32(RNG.normal(0, 1, 100))
    assert np.array_equal(lo.add(a, b), a + b)
    assert np.array_equal(lo.mul(a, b), a * b)


def test_embedding_gather_and_oob():
    W = f32(RNG.normal(0, 1, (10, 4)))
    rc, out = lo.embedding(W, [3.0, 0.0, 9.0, 3.0])
    assert rc == lo.LO_OK and np.array_equal(out, W[[3, 0, 9, 3]])
    assert lo.embedding(W, [10.0])[0] == lo.LO_ERR_EMBED_OOB                    # embedding.rs:55
    rc, out = lo.embedding(W, [2.9])                                            # `as usize` truncates
    assert rc == lo.LO_OK and np.array_equal(out[0], W[2])
    rc, out = lo.embedding(W, [-1.0])                                           # `as usize` saturates to 0
    assert rc == lo.LO_OK and np.array_equal(out[0], W[0])


def test_bf16_round_trip_matches_torch():
    x = f32(np.concatenate([RNG.normal(0, 0.02, 4096), [0.0, 1.0, -1.0, 3.0e38, 1e-40]]))
    bits = lo.f32_to_bf16(x)
    tb = torch.from_numpy(x).to(torch.bfloat16)
    assert np.array_equal(bits, tb.view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(lo.bf16_to_f32(bits), tb.float().numpy())


def test_argmax_lowest_index_on_ties():
    assert lo.argmax(f32([1, 5, 5, 2])) == 1
    assert lo.argmax(f32([-3, -3])) == 0
