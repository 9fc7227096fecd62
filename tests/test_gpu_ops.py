"""GPU parity: GEMV / GEMM / RMSNorm / elementwise / embedding / argmax / RoPE against the CPU oracle.

Tolerances: GEMV and GEMM max|d|/max|ref| <= 1e-5 (the GEMV microbenchmark's stated bound);
RoPE, add, mul and gathers bit-exact; SiLU / RMSNorm within a few f32 ulp.
"""
import numpy as np
import pytest

from lumen_amd import _lib, ops
from lumen_amd._lib import check, lib
from lumen_amd.autograd import Tensor
from lumen_amd.layers import Embedding, Linear, RMSNorm, RotaryEmbedding, SiLU
from oracle import lumen_oracle as lo
from tests.gpu_util import dev, f32, max_rel

pytestmark = pytest.mark.gpu
RNG = np.random.default_rng(99)

MICROBENCH = [(2048, 2048), (2048, 256), (2048, 5632), (5632, 2048), (2048, 32000), (4096, 11008), (11008, 4096)]


@pytest.mark.parametrize("K,N", MICROBENCH)
def test_gemv_microbench_shapes(K, N):
    rng = np.random.default_rng(K * 100003 + N)
    W = f32(rng.standard_normal((N, K), dtype=np.float32) * 0.02)  # logical (K, N), stored [N, K]
    x = f32(rng.standard_normal(K, dtype=np.float32))
    y = ops.matmul(dev(x.reshape(1, 1, K)), dev(W)).data().reshape(-1)
    ref = lo.gemv(W, x)
    assert max_rel(y, ref) <= 1e-5
    ref64 = W.astype(np.float64) @ x.astype(np.float64)
    assert max_rel(y, ref64) <= 1e-5


@pytest.mark.parametrize("N,K", [(1, 4), (3, 8), (5, 260), (7, 1000), (64, 12), (33, 37), (2, 1), (130, 513), (9, 20000)])
def test_gemv_ragged_shapes(N, K):
    W = f32(RNG.normal(0, 1, (N, K)))
    x = f32(RNG.normal(0, 1, K))
    y = Linear(dev(W)).forward(dev(x.reshape(1, K))).data().reshape(-1)
    assert max_rel(y, lo.gemv(W, x)) <= 1e-5


def test_gemv_known_answers():
    K = 512
    x = f32(RNG.normal(0, 1, K))
    assert np.array_equal(ops.matmul(dev(x[None]), dev(np.eye(K, dtype=np.float32))).data()[0], x)
    e = np.zeros(K, np.float32)
    e[77] = 1.0
    W = f32(RNG.normal(0, 1, (40, K)))
    assert np.array_equal(ops.matmul(dev(e[None]), dev(W)).data()[0], W[:, 77])


@pytest.mark.parametrize("N,K", [(256, 2048), (100, 520), (11, 8), (6, 1003)])
def test_gemv_bf16_weights(N, K):
    W = f32(RNG.normal(0, 0.02, (N, K)))
    bits = lo.f32_to_bf16(W)
    x = f32(RNG.normal(0, 1, K))
    y = ops.matmul(dev(x[None]), dev(bits)).data()[0]
    ref = lo.gemv(lo.bf16_to_f32(bits), x)  # the reference's side: same bf16 values widened (loader.rs:58)
    assert max_rel(y, ref) <= 1e-5


def test_matmul_shape_errors_and_empty():
    a = dev(np.zeros((1, 7), np.float32))
    with pytest.raises(_lib.LumenError) as e:
        ops.matmul(a, dev(np.zeros((5, 8), np.float32)))
    assert e.value.status == _lib.ERR_SHAPE
    with pytest.raises(_lib.LumenError) as e:
        ops.matmul(a, dev(np.zeros((2, 2, 2), np.float32)))
    assert e.value.status == _lib.ERR_SHAPE
    out = ops.matmul(dev(np.zeros((0, 8), np.float32)), dev(np.zeros((5, 8), np.float32)))
    assert out.shape == (0, 5)


@pytest.mark.parametrize("M,N,K", [(2, 3, 4), (7, 33, 132), (128, 256, 2048), (130, 200, 64), (64, 5632, 512),
                                   (5, 9, 7), (300, 129, 260), (16, 2560, 2048),
                                   # two rows: the vector-ALU weight-streaming kernel (whole rows per wavefront), three
                                   # and four: the matrix-core one; ragged N, K not a whole number of pieces / blocks
                                   (2, 2560, 2048), (3, 2047, 5632), (4, 11264, 2048), (4, 33, 8200), (2, 5, 1028),
                                   (4, 4096, 11008)])
def test_gemm_against_oracle(M, N, K):
    A = f32(RNG.normal(0, 1, (1, M, K)))
    W = f32(RNG.normal(0, 0.02, (N, K)))
    C = ops.matmul(dev(A), dev(W)).data()[0]
    assert C.shape == (M, N)
    ref = lo.gemm(A[0], W)
    assert max_rel(C, ref) <= 1e-5
    assert max_rel(C, A[0].astype(np.float64) @ W.T.astype(np.float64)) <= 1e-5


def test_gemm_keeps_f32_accuracy_across_magnitudes():
    """The prompt-pass product runs on the bf16 matrix cores with every f32 operand taken as three bf16 parts;
    that must not cost accuracy whatever the magnitudes: rows of A and of W scaled by powers of ten from 1e-12 to
    1e12, entries of one row spread over six decades, exact cancellation, and each output compared with the fp64
    product relative to the size of its own terms (sum |a||w|), where an f32 dot product of this length is good
    to a few 1e-7."""
    M, N, K = 96, 160, 512
    A = RNG.normal(0, 1, (M, K)) * 10.0 ** RNG.uniform(-3, 3, (M, K))
    W = RNG.normal(0, 1, (N, K)) * 10.0 ** RNG.uniform(-3, 3, (N, K))
    A *= 10.0 ** RNG.integers(-12, 13, (M, 1))
    W *= 10.0 ** RNG.integers(-12, 13, (N, 1))
    A[5, 1::2] = -A[5, 0::2]          # row 5 against row 7 of W cancels exactly
    W[7, 1::2] = W[7, 0::2]
    A, W = f32(A), f32(W)
    C = ops.matmul(dev(A[None]), dev(W)).data()[0]
    a64, w64 = A.astype(np.float64), W.astype(np.float64)
    ref, size = a64 @ w64.T, np.abs(a64) @ np.abs(w64).T
    assert np.isfinite(C).all()
    err = np.abs(C - ref) / size
    assert err.max() <= 1e-6, err.max()
    assert abs(C[5, 7]) <= 1e-6 * size[5, 7]
    # bf16-stored weights: the weight is one part, the activation still three
    bits = lo.f32_to_bf16(W)
    Wb = lo.bf16_to_f32(bits)
    Cb = ops.matmul(dev(A[None]), dev(bits)).data()[0]
    errb = np.abs(Cb - a64 @ Wb.astype(np.float64).T) / (np.abs(a64) @ np.abs(Wb.astype(np.float64)).T)
    assert errb.max() <= 1e-6, errb.max()


@pytest.mark.parametrize("M,N,K", [(5, 40, 36), (17, 96, 4), (31, 2047, 2048), (32, 2560, 2048), (9, 100, 260),
                                   (24, 11264, 2048), (32, 2048, 5632), (20, 31, 8196), (16, 48, 64)])
def test_gemm_five_to_32_rows(M, N, K):
    """Three to 32 rows of A with f32 weights: the weight-streaming matrix-core kernel (a wavefront per 16 rows of W and
    range of K, blocks of 32 k, the last one partial; one or two row tiles of A, f32 matrix instructions; ranges of K
    added inside the workgroup and, split further, in a second pass).  Values against the checker and the fp64 product, and -- rows of A and W
    scaled over 24 decades -- every output relative to the size of its own terms, as for the tile kernels."""
    A = f32(RNG.normal(0, 1, (M, K)))
    W = f32(RNG.normal(0, 0.02, (N, K)))
    C = ops.matmul(dev(A), dev(W)).data()
    assert C.shape == (M, N)
    assert max_rel(C, lo.gemm(A, W)) <= 1e-5
    assert max_rel(C, A.astype(np.float64) @ W.T.astype(np.float64)) <= 1e-5
    A2 = RNG.normal(0, 1, (M, K)) * 10.0 ** RNG.uniform(-3, 3, (M, K)) * 10.0 ** RNG.integers(-12, 13, (M, 1))
    W2 = RNG.normal(0, 1, (N, K)) * 10.0 ** RNG.uniform(-3, 3, (N, K)) * 10.0 ** RNG.integers(-12, 13, (N, 1))
    A2, W2 = f32(A2), f32(W2)
    C2 = ops.matmul(dev(A2), dev(W2)).data()
    a64, w64 = A2.astype(np.float64), W2.astype(np.float64)
    err = np.abs(C2 - a64 @ w64.T) / (np.abs(a64) @ np.abs(w64).T)
    assert np.isfinite(C2).all() and err.max() <= 1e-6, err.max()


@pytest.mark.parametrize("M,N,K", [(48, 300, 256), (3, 301, 1024), (4, 4096, 11008),
                                   # five to 32 rows: the weight-streaming matrix-core kernel, bf16 bits widened on the way
                                   (5, 40, 40), (17, 301, 1032), (32, 4096, 2048), (16, 31, 8)])
def test_gemm_bf16_weights(M, N, K):
    A = f32(RNG.normal(0, 1, (M, K)))
    bits = lo.f32_to_bf16(f32(RNG.normal(0, 0.02, (N, K))))
    C = ops.matmul(dev(A), dev(bits)).data()
    assert max_rel(C, lo.gemm(A, lo.bf16_to_f32(bits))) <= 1e-5


@pytest.mark.parametrize("M,N,K,bf16", [
    (1030, 13000, 528, False),   # 5 x 51 large tiles, no K split; ragged rows and columns, an odd number of slices
    (1100, 2816, 2048, False),   # 55 large tiles: K split in four, partial tiles added in a second pass
    (1024, 7424, 1040, True),    # bf16-stored weight, K split in two unequal shares (33 and 32 slices)
    (1500, 10496, 272, True),    # bf16-stored weight, no K split, 17 slices
])
def test_gemm_with_a_thousand_rows_and_more(M, N, K, bf16):
    """From 1024 rows of A on the product may run on 256x256 tiles (one workgroup per compute unit, K split up to
    four ways): same values as the fp64 product to 1e-5 of the largest element, and every row equal to the
    vector-matrix product of that row alone (src/ops/matmul.rs:42-69 against :70-92) within the same bound."""
    A = f32(RNG.normal(0, 1, (M, K)))
    W = f32(RNG.normal(0, 0.02, (N, K)))
    if bf16:
        bits = lo.f32_to_bf16(W)
        W = lo.bf16_to_f32(bits)
        C = ops.matmul(dev(A[None]), dev(bits)).data()[0]
    else:
        C = ops.matmul(dev(A[None]), dev(W)).data()[0]
    assert C.shape == (M, N) and np.isfinite(C).all()
    ref = A.astype(np.float64) @ W.astype(np.float64).T
    assert max_rel(C, ref) <= 1e-5
    # per element, against the size of its own terms: an f32 dot product of this length is good to a few 1e-7
    size = np.abs(A).astype(np.float64) @ np.abs(W).astype(np.float64).T
    assert (np.abs(C - ref) / size).max() <= 1e-6
    Wd = dev(bits) if bf16 else dev(W)
    for row in (0, 255, 256, M - 1):
        y = ops.matmul(dev(A[row][None]), Wd).data()[0]
        assert max_rel(C[row], y) <= 1e-5


@pytest.mark.parametrize("rows,dim,eps", [(1, 2048, 1e-5), (7, 100, 1e-6), (128, 2048, 1e-5), (3, 1, 1e-5)])
def test_rmsnorm(rows, dim, eps):
    x = f32(RNG.normal(0, 2, (rows, dim)))
    w = f32(RNG.normal(1, 0.2, dim))
    out = RMSNorm(dim, eps, w).forward(dev(x)).data()
    assert np.allclose(out, lo.rmsnorm(x, w, eps), rtol=3e-6, atol=1e-7)


def test_elementwise_and_swiglu():
    x = f32(np.concatenate([RNG.normal(0, 3, 5000), [0.0, -100.0, 100.0, -20.0, 20.0]]))
    y = f32(RNG.normal(0, 1, x.size))
    assert np.allclose(SiLU().forward(dev(x)).data(), lo.silu(x), rtol=3e-6, atol=1e-30)
    assert np.array_equal((dev(x) + dev(y)).data(), lo.add(x, y))
    assert np.array_equal((dev(x) * dev(y)).data(), lo.mul(x, y))
    assert np.allclose(ops.swiglu(dev(x), dev(y)).data(), lo.mul(lo.silu(x), y), rtol=3e-6, atol=1e-30)
    with pytest.raises(_lib.LumenError):
        dev(x) + dev(y[:10])
    assert (dev(x[:0]) + dev(y[:0])).data().size == 0


def test_embedding_and_argmax():
    W = f32(RNG.normal(0, 1, (50, 24)))
    emb = Embedding(dev(W))
    ids = np.array([[3.0, 0.0, 49.0, 3.0, 2.9]], np.float32)
    assert np.array_equal(emb.forward(ids).data(), lo.embedding(W, ids)[1])
    with pytest.raises(_lib.LumenError) as e:
        emb.forward(np.array([50.0], np.float32))
    assert e.value.status == _lib.ERR_EMBED_OOB
    v = f32(RNG.normal(0, 1, 32000))
    v[[123, 20000]] = 9.0
    assert ops.argmax(dev(v)) == lo.argmax(v) == 123
    assert ops.argmax(dev(f32([-1.0]))) == 0


@pytest.mark.parametrize("dim,max_seq,theta", [(64, 2048, 10000.0), (128, 300, 1.0e6), (16, 32, 10000.0)])
def test_rope_tables_and_rotation_bit_exact(dim, max_seq, theta):
    rope = RotaryEmbedding(dim, max_seq, theta)
    cos, sin = rope.tables()
    ocos, osin = lo.rope_table(dim, max_seq, theta)
    assert np.array_equal(cos, ocos) and np.array_equal(sin, osin)
    x = f32(RNG.normal(0, 1, (1, 3, 5, dim)))
    off = max_seq - 5
    assert np.array_equal(rope.forward(dev(x), off).data(), lo.rope_forward(x, ocos, osin, off)[1])
    with pytest.raises(_lib.LumenError) as e:
        rope.forward(dev(x), off + 1)
    assert e.value.status == _lib.ERR_ROPE_RANGE
    src = f32(RNG.normal(0, 1, dim))
    dst = Tensor.empty((dim,))
    rope.rope_1token_copy(dev(src), dst, 7)
    assert np.array_equal(dst.data(), lo.rope_1token_copy(src, ocos, osin, 7)[1])
    with pytest.raises(_lib.LumenError) as e:
        rope.rope_1token_copy(dev(src), dst, max_seq)
    assert e.value.status == _lib.ERR_ROPE_RANGE


@pytest.mark.parametrize("N,K,bf16", [(2048, 2048, False), (2048, 5632, False), (64, 512, False), (100, 264, False),
                                      (512, 1024, True), (30, 4096, True)])
def test_fused_product_equals_its_leaves(N, K, bf16):
    """lumen_gemv_fused_f32: RMSNorm on the way in and the residual / SwiGLU epilogues against the leaf operators
    of the checker (rms_norm.rs:45-58, matmul.rs:42-69, arithmetic.rs:48-51, llama.rs:59-65); gate/up rows are
    interleaved on the device with lumen_interleave_rows."""
    rng = np.random.default_rng(N * 7 + K)
    ctx = dev(np.zeros(4, np.float32)).ctx
    x = f32(rng.normal(0, 1, K))
    g = f32(rng.normal(1, 0.2, K))
    res = f32(rng.normal(0, 1, N))
    W = f32(rng.normal(0, 0.05, (N, K)))
    Wh = lo.f32_to_bf16(W) if bf16 else W
    Wref = lo.bf16_to_f32(Wh) if bf16 else W
    xd, gd, rd, Wd = dev(x), dev(g), dev(res), dev(Wh)
    eps = 1e-5
    xn = lo.rmsnorm(x[None], g, eps)[0]
    y = Tensor.empty((N,))

    def run(norm, epi, residual, out, w=Wd, n=N):
        check(lib.lumen_gemv_fused_f32(ctx.handle, w.ptr, int(bf16), xd.ptr, out.ptr, n, K, gd.ptr if norm else None, eps,
                                       epi, residual.ptr if residual is not None else None))
        return out.data()

    assert max_rel(run(False, _lib.GEMV_EPI_STORE, None, y), lo.gemv(Wref, x)) <= 1e-5
    assert max_rel(run(True, _lib.GEMV_EPI_STORE, None, y), lo.gemv(Wref, xn)) <= 1e-5
    assert max_rel(run(False, _lib.GEMV_EPI_RESIDUAL, rd, y), lo.add(res, lo.gemv(Wref, x))) <= 1e-5
    assert max_rel(run(True, _lib.GEMV_EPI_RESIDUAL, rd, y), lo.add(res, lo.gemv(Wref, xn))) <= 1e-5
    if N % 2 == 0:
        # SwiGLU: gate = first N/2 rows, up = the rest, interleaved on the device
        half = N // 2
        gate, up = Wh[:half], Wh[half:]
        gdv, udv = dev(gate), dev(up)
        Wi = Tensor.empty((N, K), Wh.dtype)
        check(lib.lumen_interleave_rows(ctx.handle, gdv.ptr, udv.ptr, Wi.ptr, half, K * Wh.itemsize))
        inter = Wi.data()
        assert np.array_equal(inter[0::2], gate) and np.array_equal(inter[1::2], up)
        act = Tensor.empty((half,))
        for norm, xin in ((False, x), (True, xn)):
            ref = lo.mul(lo.silu(lo.gemv(Wref[:half], xin)), lo.gemv(Wref[half:], xin))
            assert max_rel(run(norm, _lib.GEMV_EPI_SWIGLU, None, act, Wi, N), ref) <= 2e-5
    with pytest.raises(_lib.LumenError) as e:
        run(False, _lib.GEMV_EPI_RESIDUAL, None, y)
    assert e.value.status == _lib.ERR_INVALID
    with pytest.raises(_lib.LumenError) as e:
        run(False, 7, None, y)
    assert e.value.status == _lib.ERR_INVALID
