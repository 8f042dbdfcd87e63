"""Pins the CPU oracle independently of its own formulas (CPU only).

The reference holds no golden vectors for this path (its tests draw unseeded random
inputs and check a tolerance), so the oracle is pinned by what the mathematics fixes:
exact integer products, data-movement cases, transpose identities, FP64 products within
the forward error bound, enumeration of the split-K slice rule, and the hand-derived
heuristics table.  Where oracle/_ref is built, the reference's own micro.cuh helpers
are compared as well.
"""
import numpy as np
import pytest

from oracle import oracle
from helpers import NN, T1, T2

RNG = np.random.default_rng(20240521)


def _ops(variant, N, M, K, ints=False):
    shA = (K, N) if variant == T1 else (N, K)
    shB = (M, K) if variant == T2 else (K, M)
    if ints:
        return (RNG.integers(-4, 5, shA).astype(np.float32),
                RNG.integers(-4, 5, shB).astype(np.float32))
    return (RNG.uniform(-1, 1, shA).astype(np.float32),
            RNG.uniform(-1, 1, shB).astype(np.float32))


def _logical(variant, A, B):
    return (A.T if variant == T1 else A), (B.T if variant == T2 else B)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 7), (17, 33, 129), (64, 48, 300)])
def test_integer_inputs_are_exact(variant, shape):
    # |a|,|b| <= 4, K <= 300: every partial sum is an integer below 2^24, so any
    # correct summation order gives exactly the int64 product.  A dropped term, a
    # wrong index or a transposed operand changes the integer result.
    N, M, K = shape
    A, B = _ops(variant, N, M, K, ints=True)
    La, Lb = _logical(variant, A, B)
    exact = La.astype(np.int64) @ Lb.astype(np.int64)
    for fn in (oracle.multiply_literal, oracle.matmul):
        C = fn(variant, A, B)
        assert np.array_equal(C.astype(np.int64), exact)
        assert np.array_equal(C, exact.astype(np.float32))
    assert np.array_equal(oracle.matmul_f64(variant, A, B), exact.astype(np.float64))


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_identity_and_one_hot_move_data_only(variant):
    n = 37
    X = RNG.uniform(-1, 1, (n, n)).astype(np.float32)
    I = np.eye(n, dtype=np.float32)
    # op(A) = X, op(B) = I  ->  C = X exactly
    A = X.T.copy() if variant == T1 else X
    assert np.array_equal(oracle.matmul(variant, A, I), X)
    # op(A) = I, op(B) = X  ->  C = X exactly
    B = X.T.copy() if variant == T2 else X
    assert np.array_equal(oracle.matmul(variant, I, B), X)
    # one-hot row selector picks row 5 of op(B)
    sel = np.zeros((1, n), np.float32)
    sel[0, 5] = 1
    A1 = sel.T.copy() if variant == T1 else sel
    assert np.array_equal(oracle.matmul(variant, A1, B)[0], X[5])


def test_all_ones_gives_K():
    for K in (1, 4, 1000, 4099):
        C = oracle.matmul(NN, np.ones((3, K), np.float32), np.ones((K, 5), np.float32))
        assert np.all(C == K)


@pytest.mark.parametrize("shape", [(5, 7, 11), (33, 20, 257), (130, 70, 64)])
def test_transposed_variants_equal_plain_product_bitwise(shape):
    # matMulT1(A,B) == matMul(A^T,B) and matMulT2(A,B) == matMul(A,B^T), element by
    # element with the same k order, hence bit-identical.
    N, M, K = shape
    A, B = _ops(NN, N, M, K)
    C = oracle.matmul(NN, A, B)
    assert np.array_equal(oracle.matmul(T1, A.T.copy(), B), C)
    assert np.array_equal(oracle.matmul(T2, A, B.T.copy()), C)
    assert np.array_equal(oracle.multiply_literal(T1, A.T.copy(), B), C)
    assert np.array_equal(oracle.multiply_literal(T2, A, B.T.copy()), C)


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("shape", [(1, 1, 5), (50, 49, 131), (257, 300, 515), (96, 520, 260)])
def test_fast_is_bitwise_the_literal_loop(variant, shape):
    A, B = _ops(variant, *shape)
    assert np.array_equal(oracle.matmul(variant, A, B), oracle.multiply_literal(variant, A, B))


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_fp32_oracle_within_forward_error_bound_of_fp64(variant):
    # |fl(sum) - sum| <= gamma_K * sum |a_k b_k| for recursive summation, gamma_K ~ K*u.
    N, M, K = 40, 52, 1000
    A, B = _ops(variant, N, M, K)
    La, Lb = _logical(variant, A, B)
    exact = La.astype(np.float64) @ Lb.astype(np.float64)
    absprod = np.abs(La).astype(np.float64) @ np.abs(Lb).astype(np.float64)
    u = 2.0 ** -24
    gamma = (K + 1) * u / (1 - (K + 1) * u)
    C = oracle.matmul(variant, A, B)
    assert np.all(np.abs(C - exact) <= gamma * absprod)
    C64 = oracle.matmul_f64(variant, A, B)
    assert np.allclose(C64, exact, rtol=1e-13, atol=1e-13)
    # and not trivially equal: FP32 accumulation does round
    assert np.abs(C - exact).max() > 0


def test_fp32_oracle_is_sequential_k_ascending():
    # 2^24 + 1 + 1 ... in FP32: adding 1.0 to 2^24 one at a time never moves it,
    # while any pairwise/blocked order would.  Pins "k ascending, one add at a time".
    K = 64
    a = np.ones((1, K), np.float32)
    b = np.ones((K, 1), np.float32)
    a[0, 0] = 2.0 ** 24
    for fn in (oracle.multiply_literal, oracle.matmul):
        assert fn(NN, a, b)[0, 0] == np.float32(2.0 ** 24)
    # descending order would give 2^24 + 63 -> rounds to 2^24 + 64
    a2 = a[:, ::-1].copy()
    assert oracle.matmul(NN, a2, b)[0, 0] == np.float32(2.0 ** 24 + 64)


def test_no_fma_contraction():
    # a*b + c with a single rounding differs from round(round(a*b) + c) here.
    a = np.float32(1 + 2.0 ** -12)
    prod_rounded = np.float32(a * a)                 # 1 + 2^-11 (the 2^-24 term is lost)
    c = np.float32(-prod_rounded)
    A = np.array([[1.0, a]], np.float32)             # k=0 contributes c, k=1 contributes a*a
    B = np.array([[c], [a]], np.float32)
    got = oracle.matmul(NN, A, B)[0, 0]
    assert got == np.float32(0.0)                    # separate rounding: exactly cancels
    assert np.float64(a) * np.float64(a) + np.float64(c) != 0.0   # a fused multiply-add would not


# ---- batched ---------------------------------------------------------------------------
def _bmm_case(variant, Batch, N, M, K):
    """Logical batched operands laid out in the reference's padded memory layout."""
    p4 = lambda v: (v + 3) // 4 * 4
    if variant == NN:      # A[B,N,AK], B[B,BK,CM]
        AK, CM = p4(K), p4(M)
        A = np.zeros((Batch, N, AK), np.float32); A[:, :, :K] = RNG.uniform(-1, 1, (Batch, N, K))
        B = np.zeros((Batch, K, CM), np.float32); B[:, :, :M] = RNG.uniform(-1, 1, (Batch, K, M))
        dims = (N, CM, K, AK)
        ref = A[:, :, :K].astype(np.float64) @ B.astype(np.float64)
    elif variant == T1:    # A[B,K,AN], B[B,K,CM] -> C[B,CN,CM]
        AN, CM = p4(N), p4(M)
        A = np.zeros((Batch, K, AN), np.float32); A[:, :, :N] = RNG.uniform(-1, 1, (Batch, K, N))
        B = np.zeros((Batch, K, CM), np.float32); B[:, :, :M] = RNG.uniform(-1, 1, (Batch, K, M))
        dims = (N, AN, CM, K)
        ref = np.transpose(A[:, :, :N], (0, 2, 1)).astype(np.float64) @ B.astype(np.float64)
    else:                  # A[B,N,K4], B[B,BM,K4] -> C[B,N,CM]
        K4, CM = p4(K), p4(M)
        A = np.zeros((Batch, N, K4), np.float32); A[:, :, :K] = RNG.uniform(-1, 1, (Batch, N, K))
        B = np.zeros((Batch, M, K4), np.float32); B[:, :, :K] = RNG.uniform(-1, 1, (Batch, M, K))
        dims = (N, CM, M, K4)
        ref = np.zeros((Batch, N, CM))
        ref[:, :, :M] = A.astype(np.float64) @ np.transpose(B, (0, 2, 1)).astype(np.float64)
    return A, B, dims, ref


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("shape", [(3, 5, 6, 7), (4, 33, 21, 9), (2, 70, 130, 50)])
def test_batched_oracle(variant, shape):
    Batch, N, M, K = shape
    A, B, dims, ref = _bmm_case(variant, Batch, N, M, K)
    C1 = oracle.bmm_literal(variant, A, B, Batch, *dims)
    C2 = oracle.bmm(variant, A, B, Batch, *dims)
    assert np.array_equal(C1, C2)
    assert np.allclose(C1, ref, rtol=0, atol=2e-5 * np.sqrt(K))
    # batched == loop of 2-D products on the logical slices, bit for bit
    for b in range(Batch):
        if variant == NN:
            c = oracle.matmul(NN, A[b][:, :K], B[b])
        elif variant == T1:
            c = oracle.matmul(T1, A[b][:, :N], B[b])
        else:
            c = np.zeros_like(C1[b])
            c[:, :M] = oracle.matmul(T2, A[b], B[b])
        assert np.array_equal(C1[b], c)


# ---- split-K -----------------------------------------------------------------------------
def test_split_k_slice_rule_enumerated():
    for K in list(range(8, 300, 4)) + [1532, 4096, 131072]:
        for GZ in (1, 2, 3, 4, 7, 16, 36, 128):
            ks = oracle.SK_K_slice(K, GZ)
            assert ks % 8 == 0 and ks == (K // GZ) // 8 * 8
            total, prev_end = 0, 0
            for z in range(GZ):
                a, b = oracle.SK_bounds(K, GZ, z)
                assert a == prev_end and b >= a
                if z < GZ - 1:
                    assert b - a == ks
                else:
                    assert b == K            # the last slice takes the remainder
                total += b - a
                prev_end = b
            assert total == K
    assert oracle.SK_K_slice(131072, 128) == 1024
    assert oracle.SK_K_slice(131072, 36) == 3640
    assert oracle.SK_K_slice(1532, 2) == 760


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_split_k_partials_sum_to_product(variant):
    N, M, K, GZ = 24, 36, 1000, 6
    A, B = _ops(variant, N, M, K, ints=True)
    La, Lb = _logical(variant, A, B)
    exact = (La.astype(np.int64) @ Lb.astype(np.int64)).astype(np.float32)
    C0, Cbuf = oracle.matMulSK(variant, GZ, A, B)
    assert Cbuf.shape == (GZ - 1, N, M)
    # each partial is the exact product over its own k range
    for z in range(GZ):
        a, b = oracle.SK_bounds(K, GZ, z)
        part = (La[:, a:b].astype(np.int64) @ Lb[a:b].astype(np.int64)).astype(np.float32)
        assert np.array_equal(C0 if z == 0 else Cbuf[z - 1], part)
    assert np.array_equal(oracle.SKbuf_summary(Cbuf, C0, GZ - 1), exact)


def test_kahan_summary_beats_plain_sum_and_matches_fp64():
    # one large value followed by many small ones: plain FP32 accumulation loses them,
    # the compensated sum keeps them.
    part, sizeC = 127, 64
    C = np.full(sizeC, 1.0e4, np.float32)
    Cbuf = RNG.uniform(1e-4, 2e-4, (part, sizeC)).astype(np.float32)
    exact = C.astype(np.float64) + Cbuf.astype(np.float64).sum(axis=0)
    got = oracle.SKbuf_summary(Cbuf, C, part)
    plain = C.copy()
    for p in range(part):
        plain = plain + Cbuf[p]
    assert np.abs(got - exact).max() <= np.spacing(np.float32(1.0e4))   # within 1 ulp
    assert np.abs(plain - exact).max() > 5 * np.abs(got - exact).max()
    # part = 0 leaves C untouched
    assert np.array_equal(oracle.SKbuf_summary(Cbuf, C, 0), C)


# ---- heuristics ------------------------------------------------------------------------------
def _tile_count_bruteforce(n):
    """Greedy carve of n (multiple of 4) into 128,64,32,16,8,4 tiles: number of tiles."""
    cnt = 0
    for t in (128, 64, 32, 16, 8, 4):
        cnt += n // t
        n %= t
    return cnt


def _class_count_bruteforce(n):
    if n & (n - 1) == 0:
        return 1
    cnt = 0
    for t in (128, 64, 32, 16, 8, 4):
        if n >= t:
            cnt += 1
        n %= t
    return cnt


def test_blockNum_and_nstream_against_bruteforce():
    for N in range(4, 1300, 4):
        for M in (4, 8, 12, 64, 100, 128, 252, 256, 780, 1000, 1028):
            assert oracle.blockNum(N, M) == _tile_count_bruteforce(N) * _tile_count_bruteforce(M)
            ns = min(10, _class_count_bruteforce(N) * _class_count_bruteforce(M))
            assert oracle.nstream(N, M) == ns
            assert oracle.streamSize(N, M) == max(1, ns)


def test_heuristics_known_answers():
    # hand-derived from the Java sources
    assert oracle.blockNum(4096, 4096) == 1024
    assert oracle.blockNum(256, 256) == 4
    assert oracle.blockNum(1000, 780) == 80
    assert oracle.blockNum(512, 512) == 16
    assert oracle.nstream(4096, 4096) == 1
    assert oracle.nstream(1000, 780) == 10
    assert oracle.smooth_maxPart(256) == 128
    assert oracle.smooth_maxPart(38) == 40
    assert oracle.smooth_maxPart(10) == 16
    assert oracle.smooth_maxPart(30) == 32
    # BASELINE shapes with 256 compute units
    for kind in (oracle.MATMUL, oracle.MATMUL_T1, oracle.MATMUL_T2):
        assert oracle.gridZ(kind, 4096, 4096, 4096, 256) == 1
        assert oracle.gridZ(kind, 1000, 780, 1532, 256) == 2
    assert oracle.gridZ(oracle.MATMUL_T1, 256, 256, 131072, 256) == 128
    # the same weight-gradient shape on a 38-SM device
    assert oracle.gridZ(oracle.MATMUL_T1, 256, 256, 131072, 38) == 36
    # below the threshold nothing splits
    assert oracle.gridZ(oracle.MATMUL, 128, 128, 508, 256) == 1


def test_matMulT2_policy_known_answers_that_need_its_quirks():
    """matMulT2 (CudaFloat32EngineBase.java:1859-1867, 1894) tests b2 = blockNum(N, K) -- not the
    blockNum(N, M) of its own output -- against matMul's constant 1.2 (matMul_sk_minBlock_perSM, not
    matMulT2_sk_minBlock_perSM = 1.14) and divides by that same b2 in the GridZ3 clamp.  Each answer below
    is derived by hand from the Java text and comes out differently when one of those is "corrected"."""
    SM = 256
    # N = M = 64, K = 8192: b2 = blockNum(64, 8192) = 1 * 64 = 64 < 256 * (1.2 + 8192/9216) = 534.8
    #   b0 = blockNum(64, 64) = 1, b1 = blockNum(8192, 64) = 64, fGridZ = (64 + 64) / 2 = 64
    #   GridZ2 = 8192 >> 8 = 32 -> 32;  GridZ3 = int(256 * 4 * (8192/12288) / 64) = int(10.67) = 10 -> 10
    #   padded to a multiple of 4: 12.   (With b0 in the clamp: GridZ3 = 682 -> 32, which is what
    #   matMulT1 answers for this shape.)
    assert oracle.blockNum(64, 8192) == 64 and oracle.blockNum(8192, 64) == 64 and oracle.blockNum(64, 64) == 1
    assert oracle.gridZ(oracle.MATMUL_T2, 64, 64, 8192, SM) == 12
    assert oracle.gridZ(oracle.MATMUL_T1, 64, 64, 8192, SM) == 32
    # K = 65536: b2 = 512 < 256 * (1.2 + 65536/66560) = 559.3; fGridZ = (512 + 512) / 2 = 512
    #   GridZ2 = 256 -> 256;  GridZ3 = int(1024 * (65536/69632) / 512) = int(1.88) = 1 -> 1 -> raised to 2.
    #   (With b0 in the clamp: 963 -> 256 -> maxPart 128, matMulT1's answer.)
    assert oracle.blockNum(64, 65536) == 512
    assert oracle.gridZ(oracle.MATMUL_T2, 64, 64, 65536, SM) == 2
    assert oracle.gridZ(oracle.MATMUL_T1, 64, 64, 65536, SM) == 128
    # The constant alone: N = 6784 (53 tiles of 128), M = 4, K = 1024: b2 = blockNum(6784, 1024) = 53 * 8 = 424
    #   lies between 256 * (1.14 + 0.5) = 419.8 and 256 * (1.2 + 0.5) = 435.2, so the product is split only
    #   because matMul's 1.2 is used: b0 = 53, b1 = blockNum(1024, 4) = 8, fGridZ = (8 + 424) / 106 = 4.08
    #   GridZ2 = 4;  GridZ3 = int(1024 * 0.2 / 424) = 0 -> raised to 2.   (With 1.14: no split, 1.)
    assert oracle.blockNum(6784, 1024) == 424 and oracle.blockNum(6784, 4) == 53 and oracle.blockNum(1024, 4) == 8
    assert oracle.gridZ(oracle.MATMUL_T2, 6784, 4, 1024, SM) == 2


def test_biased_policy_known_answer():
    # hand-derived (see the arithmetic in test_host_policy.test_known_answers)
    assert oracle.blockNum(2048, 4096) == 512
    assert oracle.gridZ(oracle.MATMUL, 2048, 4096, 16384, 256) == 1
    assert oracle.gridZ(oracle.MATMUL_BIASED, 2048, 4096, 16384, 256) == 2
    # where both split they agree: the clamp is shared
    assert oracle.gridZ(oracle.MATMUL_BIASED, 1000, 780, 1532, 256) == 2


def test_bias_row_is_an_exact_add_and_zeroes_the_pad():
    rows, width = 37, 50
    stride = 52
    X1 = np.zeros((rows, stride), np.float32)
    X1[:, :width] = RNG.uniform(-3, 3, (rows, width)).astype(np.float32)
    X1[:, width:] = 7.0            # garbage in the pad must come out as zero
    X2 = np.zeros(stride, np.float32)
    X2[:width] = RNG.uniform(-1, 1, width).astype(np.float32)
    Y = oracle.linear_dual2D_row(X1, X2, 1.0, 1.0, 0.0, width)
    assert np.array_equal(Y[:, :width], X1[:, :width] + X2[None, :width])   # numpy adds in float32
    assert np.all(Y[:, width:] == 0)
    # integers: exact whatever the rounding order
    Xi = RNG.integers(-100, 100, (8, 8)).astype(np.float32)
    bi = RNG.integers(-100, 100, 8).astype(np.float32)
    Yi = oracle.linear_dual2D_row(Xi, bi, 3.0, -2.0, 5.0, 8)
    assert np.array_equal(Yi, 3 * Xi - 2 * bi[None, :] + 5)


def test_bias_row_general_coefficients_within_rounding_of_fp64():
    rows, width, stride = 64, 33, 36
    X1 = np.zeros((rows, stride), np.float32)
    X1[:, :width] = RNG.normal(size=(rows, width)).astype(np.float32)
    X2 = np.zeros(stride, np.float32)
    X2[:width] = RNG.normal(size=width).astype(np.float32)
    a, b, g = np.float32(0.37), np.float32(-1.91), np.float32(0.123)
    Y = oracle.linear_dual2D_row(X1, X2, a, b, g, width)
    ref = np.float64(a) * X1.astype(np.float64) + np.float64(b) * X2.astype(np.float64)[None, :] + np.float64(g)
    mag = np.abs(np.float64(a) * X1) + np.abs(np.float64(b) * X2)[None, :] + abs(np.float64(g))
    # four roundings, each at most half an ulp of a partial result no larger than mag
    assert np.all(np.abs(Y[:, :width] - ref[:, :width]) <= 4 * 2.0 ** -24 * mag[:, :width])
    assert np.all(Y[:, width:] == 0)


def _dev_layout(X):
    s = (X.shape[-1] + 3) // 4 * 4
    out = np.zeros(X.shape[:-1] + (s,), np.float32)
    out[..., :X.shape[-1]] = X
    return out


@pytest.mark.parametrize("dims,i1,i2", [((5, 7), 0, 1), ((4, 8), 1, 0), ((2, 3, 5), 1, 2), ((2, 3, 5), 0, 2),
                                        ((2, 3, 5), 0, 1), ((2, 3, 4, 6), 1, 2), ((2, 3, 4, 6), 0, 3),
                                        ((2, 3, 4, 6), 2, 3), ((3, 1, 2, 9), 1, 3), ((1, 1), 0, 1)])
def test_transpose_oracle_is_numpy_swapaxes_and_an_involution(dims, i1, i2):
    X = RNG.standard_normal(dims).astype(np.float32)
    Yp = oracle.transpose(_dev_layout(X), dims, i1, i2)
    Y = np.swapaxes(X, i1, i2)
    assert Yp.shape[:-1] == Y.shape[:-1] and Yp.shape[-1] == (Y.shape[-1] + 3) // 4 * 4
    assert np.array_equal(Yp[..., :Y.shape[-1]], Y)        # every element where numpy puts it
    assert not Yp[..., Y.shape[-1]:].any()                 # pad untouched (zero)
    back = oracle.transpose(Yp, list(Y.shape), i1, i2)     # swapping twice restores the layout
    assert np.array_equal(back, _dev_layout(X))


def test_softmax_oracle_against_fp64_and_its_invariants():
    rows, width, stride = 40, 37, 40
    X = np.zeros((rows, stride), np.float32)
    X[:, :width] = RNG.standard_normal((rows, width)).astype(np.float32) * 3
    X[:, width:] = 50.0                                 # garbage in the pad must not take part
    Y = oracle.softmax2D(X, width)
    e = np.exp(X[:, :width].astype(np.float64) - X[:, :width].astype(np.float64).max(1, keepdims=True))
    R = e / e.sum(1, keepdims=True)
    # x - max rounded to float (an absolute error of up to 2^-25 |x - max| in the exponent), exp within an
    # ulp, a float sum of 37 terms, one division
    dist = np.abs(X[:, :width].astype(np.float64) - X[:, :width].astype(np.float64).max(1, keepdims=True))
    assert np.all(np.abs(Y[:, :width] - R) <= 2.0 ** -24 * (dist + 8) * R + 1e-38)
    assert not Y[:, width:].any()
    assert np.allclose(Y.sum(1), 1.0, atol=3e-7)
    # equal inputs over a power-of-two count give exactly 1/n; one element gives exactly 1
    U = np.full((3, 8), 2.5, np.float32)
    assert np.array_equal(oracle.softmax2D(U, 8), np.full((3, 8), 0.125, np.float32))
    one = np.zeros((5, 4), np.float32); one[:, 0] = RNG.standard_normal(5)
    assert np.array_equal(oracle.softmax2D(one, 1)[:, 0], np.ones(5, np.float32))
    # a dominant element: exp underflows to an exact zero next to an exact one
    D = np.zeros((1, 4), np.float32); D[0, :3] = [0.0, 200.0, -5.0]
    assert np.array_equal(oracle.softmax2D(D, 3)[0, :3], np.array([0.0, 1.0, 0.0], np.float32))
    # features spanning two memory rows: softmax over both rows' logical elements together
    Y2 = oracle.softmax2D(X, width, features=2 * width)
    e2 = np.exp(X[:, :width].astype(np.float64).reshape(rows // 2, 2 * width))
    R2 = (e2 / e2.sum(1, keepdims=True)).reshape(rows, width)
    assert np.all(np.abs(Y2[:, :width] - R2) <= 1e-6 * R2 + 1e-38)
    # the scale is the same as scaling the input first (power of two: exact)
    assert np.array_equal(oracle.softmax2D(X, width, scale=0.5), oracle.softmax2D(X * np.float32(0.5), width))


def test_linear2D_oracle():
    X = np.zeros((6, 8), np.float32); X[:, :7] = RNG.integers(-9, 9, (6, 7))
    X[:, 7] = 3.0
    Y = oracle.linear2D(2.0, X, -1.0, 7)
    assert np.array_equal(Y[:, :7], 2 * X[:, :7] - 1) and not Y[:, 7].any()


def _conv_numpy(X, W, sh, sw, ph, pw):
    """Independent restatement: zero-pad, gather windows with stride tricks, contract with einsum in FP64."""
    N, IH, IW, IC = X.shape
    OC, FH, FW, _ = W.shape
    Xp = np.zeros((N, IH + 2 * ph, IW + 2 * pw, IC), np.float64)
    Xp[:, ph:ph + IH, pw:pw + IW] = X
    OH, OW = (IH - FH + 2 * ph) // sh + 1, (IW - FW + 2 * pw) // sw + 1
    win = np.lib.stride_tricks.sliding_window_view(Xp, (FH, FW), axis=(1, 2))[:, ::sh, ::sw][:, :OH, :OW]
    return np.einsum("nhwcij,oijc->nhwo", win, W.astype(np.float64))


@pytest.mark.parametrize("geom", [(5, 5, 3, 3, 1, 1, 1, 1), (8, 7, 3, 3, 2, 2, 1, 1), (9, 9, 4, 4, 1, 1, 1, 1),
                                  (6, 6, 1, 1, 1, 1, 0, 0), (7, 9, 3, 2, 2, 1, 0, 0), (4, 4, 4, 4, 1, 1, 3, 3),
                                  (10, 6, 5, 3, 3, 2, 2, 1)])
def test_conv_oracle_against_an_independent_formulation(geom):
    IH, IW, FH, FW, sh, sw, ph, pw = geom
    N, IC, OC = 2, 3, 5
    X = RNG.standard_normal((N, IH, IW, IC)).astype(np.float32)
    W = RNG.standard_normal((OC, FH, FW, IC)).astype(np.float32)
    Y = oracle.conv3D(X, W, sh, sw, ph, pw)
    R = _conv_numpy(X, W, sh, sw, ph, pw)
    assert Y.shape == R.shape
    assert np.array_equal(Y, R.astype(np.float32))          # FP64 accumulation rounded once: same floats
    # integer inputs: the float accumulator variant is exact too
    Xi = RNG.integers(-3, 4, X.shape).astype(np.float32)
    Wi = RNG.integers(-3, 4, W.shape).astype(np.float32)
    assert np.array_equal(oracle.conv3D(Xi, Wi, sh, sw, ph, pw, acc32=True), _conv_numpy(Xi, Wi, sh, sw, ph, pw))


def test_conv_oracle_special_cases():
    # a 1x1 filter is a matrix product over the channels
    X = RNG.standard_normal((2, 4, 5, 6)).astype(np.float32)
    W = RNG.standard_normal((7, 1, 1, 6)).astype(np.float32)
    Y = oracle.conv3D(X, W, 1, 1, 0, 0)
    assert np.allclose(Y.reshape(-1, 7), X.reshape(-1, 6).astype(np.float64) @ W.reshape(7, 6).T.astype(np.float64),
                       rtol=1e-6, atol=1e-6)
    # a one-hot filter copies a shifted channel; the border comes from the zero padding
    W1 = np.zeros((1, 3, 3, 6), np.float32); W1[0, 0, 2, 4] = 1.0        # picks X[ih-1, iw+1, channel 4]
    Y1 = oracle.conv3D(X, W1, 1, 1, 1, 1)[..., 0]
    exp = np.zeros_like(Y1); exp[:, 1:, :-1] = X[:, :-1, 1:, 4]
    assert np.array_equal(Y1, exp)
    # linear in W
    Wa = RNG.standard_normal((3, 3, 3, 6)).astype(np.float32)
    Wb = RNG.standard_normal((3, 3, 3, 6)).astype(np.float32)
    ya, yb = oracle.conv3D(X, Wa, 2, 1, 1, 0), oracle.conv3D(X, Wb, 2, 1, 1, 0)
    assert np.allclose(oracle.conv3D(X, Wa + Wb, 2, 1, 1, 0), ya + yb, rtol=1e-5, atol=1e-5)


def test_attention_oracle_is_the_chain_and_matches_fp64():
    # oracle.attention composes the pinned batched products, linear2D and softmax2D the way the reference's
    # block does; against the same mathematics in FP64, and on cases with a known answer
    for (B, QL, VL, dk, dv, alpha) in [(3, 5, 9, 7, 6, 0.3), (2, 33, 65, 20, 12, 0.125), (1, 1, 1, 1, 1, 2.0),
                                       (2, 17, 40, 64, 64, -0.5)]:
        Q = RNG.standard_normal((B, QL, dk)).astype(np.float32)
        K = RNG.standard_normal((B, VL, dk)).astype(np.float32)
        V = RNG.standard_normal((B, VL, dv)).astype(np.float32)
        Y = oracle.attention(Q, K, V, alpha)
        S = np.einsum("bqd,bkd->bqk", Q.astype(np.float64), K.astype(np.float64)) * np.float64(np.float32(alpha))
        P = np.exp(S - S.max(-1, keepdims=True))
        P /= P.sum(-1, keepdims=True)
        R = np.einsum("bqk,bkd->bqd", P, V.astype(np.float64))
        assert Y.shape == R.shape
        assert np.abs(Y - R).max() <= 1e-5 * max(1.0, np.abs(V).max()), (B, QL, VL)
    V = RNG.standard_normal((1, 9, 4)).astype(np.float32)
    Y = oracle.attention(np.zeros((1, 3, 5), np.float32), RNG.standard_normal((1, 9, 5)).astype(np.float32), V, 1.0)
    assert np.abs(Y - V.astype(np.float64).mean(1)).max() <= 1e-6          # equal scores: the mean of V
    Q = np.zeros((1, 2, 4), np.float32); Q[..., 0] = 60.0
    K = np.zeros((1, 9, 4), np.float32); K[0, 6, 0] = 1.0
    assert np.abs(oracle.attention(Q, K, V, 1.0) - V[0, 6]).max() <= 1e-6   # one key dominates: its row of V


def test_attention_oracle_applies_the_mask_after_the_softmax():
    # ChannelMHA.java:74-78: P = softmax(...); if (mask != null) P = mask.forward(P) -- the mask multiplies the
    # probabilities, the rows are NOT normalised again.  Against that mathematics in FP64, and on cases that a
    # mask applied before the softmax (the other common convention) would get wrong.
    B, QL, VL, dk, dv, alpha = 2, 7, 13, 8, 5, 0.4
    Q = RNG.standard_normal((B, QL, dk)).astype(np.float32)
    K = RNG.standard_normal((B, VL, dk)).astype(np.float32)
    V = RNG.standard_normal((B, VL, dv)).astype(np.float32)
    ones = np.ones((QL, VL), np.float32)
    assert np.array_equal(oracle.attention(Q, K, V, alpha, mask=ones), oracle.attention(Q, K, V, alpha))
    causal = np.tril(np.ones((QL, VL), np.float32))
    per_entry = RNG.uniform(0, 2, (B, QL, VL)).astype(np.float32)
    S = np.einsum("bqd,bkd->bqk", Q.astype(np.float64), K.astype(np.float64)) * np.float64(np.float32(alpha))
    P = np.exp(S - S.max(-1, keepdims=True))
    P /= P.sum(-1, keepdims=True)
    for M in (causal, per_entry):
        R = np.einsum("bqk,bkd->bqd", P * np.broadcast_to(M, P.shape), V.astype(np.float64))
        assert np.abs(oracle.attention(Q, K, V, alpha, mask=M) - R).max() <= 1e-5 * max(1.0, np.abs(V).max())
    # a zero on the one key that holds all the probability: the output is (nearly) zero, where masking the
    # score before the softmax would have handed the weight to the other keys
    Q = np.zeros((1, 1, 4), np.float32); Q[..., 0] = 60.0
    K = np.zeros((1, 9, 4), np.float32); K[0, 6, 0] = 1.0
    V = np.ones((1, 9, 3), np.float32)
    M = np.ones((1, 9), np.float32); M[0, 6] = 0.0
    assert np.abs(oracle.attention(Q, K, V, 1.0, mask=M)).max() <= 1e-6
    # a zero mask gives exact zeros; a mask of twos doubles the output exactly
    assert not oracle.attention(Q, K, V, 1.0, mask=np.zeros((1, 9), np.float32)).any()
    Y1 = oracle.attention(Q, K, V, 1.0)
    assert np.array_equal(oracle.attention(Q, K, V, 1.0, mask=2 * np.ones((1, 9), np.float32)), 2 * Y1)


def test_reference_micro_helpers_when_built():
    ref = oracle.load_ref()
    if ref is None:
        pytest.skip("oracle/_ref is not built (reference tree absent at build time)")
    for N in range(4, 1100, 4):
        for M in (4, 60, 128, 388, 780, 1024):
            assert ref.ref_blockNum(N, M) == oracle.blockNum(N, M)
    for K in (8, 100, 1532, 4096, 131072):
        for GZ in (1, 2, 5, 36, 128):
            assert ref.ref_SK_K_slice(K, GZ) == oracle.SK_K_slice(K, GZ)


def test_samePercent_relative_rule():
    a = np.array([1.0, 2.0, 0.0, 5.0, np.nan], np.float32)
    b = np.array([1.0005, 2.1, 0.0, 5.0, np.nan], np.float32)
    # 1.0 vs 1.0005: 2.5e-4 < 1e-3 same; 2.0 vs 2.1: 2.4e-2 different; equal; equal; NaN pair same
    assert oracle.samePercent_relative(a, b) == pytest.approx(4 / 5)
