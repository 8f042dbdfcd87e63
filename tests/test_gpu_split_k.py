"""GPU parity of the two-stage split-K path (matMul*SK + SKbuf_summary)."""
import numpy as np
import pytest

from oracle import oracle
from helpers import NN, T1, T2, VARIANT_NAMES, assert_within_tolerance, gpu_matmul_2d, logical_operands, pad2, rel_fro

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _slices_as_asked(gpu):
    """The tests of the slice rule need the slices: the entry points are told to honour every GridZ (they
    otherwise decline a split they estimate to lose; that behaviour has tests of its own below)."""
    gpu.split_policy(0)
    yield
    gpu.split_policy(-1)
    gpu.force_tile(-1)


def run_sk(gpu, variant, A, B, GZ, summary=True, fill=9.0):
    """A, B already padded to x4.  Returns (C, Cbuf) as written by stage 1 (and stage 2)."""
    MM, Cuda = gpu.Cuda_matMul, gpu.Cuda
    if variant == NN:
        (N, K), M = A.shape, B.shape[1]
    elif variant == T1:
        (K, N), M = A.shape, B.shape[1]
    else:
        (N, K), M = A.shape, B.shape[0]
    dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
    dC, dCbuf = gpu.DeviceArray(size=N * M), gpu.DeviceArray(size=N * M * max(GZ - 1, 1))
    dC.fill(fill)
    dCbuf.fill(fill)
    [MM.matMulSK, MM.matMulT1SK, MM.matMulT2SK][variant]([0], 1, GZ, dA.address, dB.address,
                                                           dC.address, dCbuf.address, N, M, K)
    if summary:
        MM.SKbuf_summary(0, dCbuf.address, dC.address, GZ - 1, N * M)
    Cuda.streamSynchronize(0)
    C, Cbuf = dC.get((N, M)), dCbuf.get((max(GZ - 1, 1), N, M))[:GZ - 1]
    for x in (dA, dB, dC, dCbuf):
        x.free()
    return C, Cbuf


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("shape_gz", [((64, 64, 256), 2), ((128, 132, 1000), 6), ((36, 260, 1532), 2),
                                      ((256, 256, 4096), 16), ((100, 52, 904), 7), ((8, 8, 40), 4)])
def test_stage1_partials_follow_the_slice_rule_bitwise(gpu, variant, shape_gz):
    # integer inputs: each slice's partial product is exact, so slice bounds that are off
    # by a single k show up as a bit mismatch against the oracle's partials
    (N, M, K), GZ = shape_gz
    rng = np.random.default_rng(K + GZ)
    A, B = logical_operands(variant, rng, N, M, K, dist="int")
    C, Cbuf = run_sk(gpu, variant, A, B, GZ, summary=False)
    C0, Cb0 = oracle.matMulSK(variant, GZ, A, B)
    assert np.array_equal(C, C0)
    assert np.array_equal(Cbuf, Cb0)
    # after stage 2 the product is complete
    C, _ = run_sk(gpu, variant, A, B, GZ, summary=True)
    assert np.array_equal(C, oracle.matmul(variant, A, B))


def test_stage2_summary_is_bit_identical_to_the_reference_order(gpu):
    rng = np.random.default_rng(77)
    MM, Cuda = gpu.Cuda_matMul, gpu.Cuda
    for part, sizeC in [(1, 4), (3, 64), (7, 252), (15, 256), (127, 65536), (33, 100004), (9, 1 << 20)]:
        C = (rng.standard_normal(sizeC) * 100).astype(np.float32)
        Cbuf = rng.standard_normal((part, sizeC)).astype(np.float32)
        Cbuf[::2] *= 1e-4                       # mixed magnitudes exercise the compensation
        dC, dCbuf = gpu.DeviceArray(C), gpu.DeviceArray(Cbuf)
        MM.SKbuf_summary(0, dCbuf.address, dC.address, part, sizeC)
        Cuda.streamSynchronize(0)
        got = dC.get()
        assert np.array_equal(got, oracle.SKbuf_summary(Cbuf, C, part)), (part, sizeC)
        exact = C.astype(np.float64) + Cbuf.astype(np.float64).sum(axis=0)
        assert np.abs(got - exact).max() <= 2 * np.spacing(np.abs(exact).max().astype(np.float32))
        dC.free(); dCbuf.free()


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_split_k_equals_unsplit_within_tolerance(gpu, variant):
    rng = np.random.default_rng(3 + variant)
    N, M, K = 256, 128, 8192
    A, B = logical_operands(variant, rng, N, M, K, dist="normal")
    R32 = oracle.matmul(variant, A, B)
    R64 = oracle.matmul_f64(variant, A, B)
    for GZ in (2, 8, 32):
        C, _ = run_sk(gpu, variant, A, B, GZ)
        assert_within_tolerance(C, R32, K, A, B, "%s GZ=%d vs FP32 oracle" % (VARIANT_NAMES[variant], GZ))
        assert_within_tolerance(C, R64, K, A, B, "%s GZ=%d vs FP64 oracle" % (VARIANT_NAMES[variant], GZ))
        # and against the oracle's own two-stage computation
        C0, Cb0 = oracle.matMulSK(variant, GZ, A, B)
        assert rel_fro(C, oracle.SKbuf_summary(Cb0, C0, GZ - 1)) < 2e-6


@pytest.mark.parametrize("tile", [1, 6, 7, 9, 10, 11, 12, 14, 15, 16, 17, 18, 19, 20, 21, 22, 23, 256, 257, 262, 263, 265])
def test_split_k_with_every_stage_depth(gpu, tile):
    # K slices that are not multiples of the k stage (16 or 32), on forced tile shapes
    rng = np.random.default_rng(50 + tile)
    gpu.force_tile(tile)
    try:
        for variant in (NN, T1, T2):
            A, B = logical_operands(variant, rng, 132, 68, 1000, dist="int")
            C, Cbuf = run_sk(gpu, variant, A, B, 6, summary=False)
            C0, Cb0 = oracle.matMulSK(variant, 6, A, B)
            assert np.array_equal(C, C0) and np.array_equal(Cbuf, Cb0)
    finally:
        gpu.force_tile(-1)


@pytest.mark.parametrize("tile", [18, 19, 20, 21, 22, 23, 25])
@pytest.mark.parametrize("shape_gz", [((300, 260, 5000), 5), ((256, 256, 4100), 3), ((64, 200, 40000), 37),
                                      ((520, 136, 2056), 2)])
def test_k_slices_through_the_balanced_kernel(gpu, tile, shape_gz):
    """The balanced kernel takes (K slice, tile) pairs as its tiles: the last slice is longer than the others
    ((256, 256, 4100) in 3: 1360, 1360, 1380), runs cross from one slice into the next, and tiles shared by
    several workgroups are put together from pieces.  Integer inputs: every partial is exact."""
    (N, M, K), GZ = shape_gz
    rng = np.random.default_rng(K + GZ + tile)
    gpu.force_tile(tile)
    try:
        for variant in (NN, T1, T2):
            A, B = logical_operands(variant, rng, N, M, K, dist="int")
            C, Cbuf = run_sk(gpu, variant, A, B, GZ, summary=False)
            C0, Cb0 = oracle.matMulSK(variant, GZ, A, B)
            assert np.array_equal(C, C0) and np.array_equal(Cbuf, Cb0), (variant, shape_gz, tile)
    finally:
        gpu.force_tile(-1)


def test_degenerate_slices(gpu):
    # K smaller than 8*GridZ: K_slice = 0, every slice but the last is empty and must be
    # written as zeros; the last carries the whole product
    rng = np.random.default_rng(11)
    A, B = logical_operands(T1, rng, 32, 36, 24, dist="int")
    C, Cbuf = run_sk(gpu, T1, A, B, 4, summary=False)
    assert oracle.SK_K_slice(24, 4) == 0
    assert np.count_nonzero(C) == 0 and np.count_nonzero(Cbuf[:2]) == 0
    assert np.array_equal(Cbuf[2], oracle.matmul(T1, A, B))
    # GridZ = 1 through the split-K entry is the plain product (Cbuf unused)
    MM = gpu.Cuda_matMul
    dA, dB, dC = gpu.DeviceArray(A), gpu.DeviceArray(B), gpu.DeviceArray(size=32 * 36)
    MM.matMulT1SK([0], 1, 1, dA.address, dB.address, dC.address, 0, 32, 36, 24)
    gpu.Cuda.streamSynchronize(0)
    assert np.array_equal(dC.get((32, 36)), oracle.matmul(T1, A, B))


# ---- a split that loses is declined: the whole product in C, exact zeros in the partial buffers ----

DECLINED = [((1000, 780, 1532), 2), ((512, 512, 4096), 2), ((1024, 768, 2048), 2)]


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("shape_gz", DECLINED)
def test_a_losing_split_is_declined(gpu, variant, shape_gz):
    """The host's policy asks for GridZ slices of a product that the balanced kernel runs faster unsplit (the
    three shapes: two 64 x 64 tiles per unit at most and a K long enough): C then holds the whole product --
    the very bits of the unsplit entry point --, every float of Cbuf is +0, and the fold leaves C as it is."""
    (N, M, K), GZ = shape_gz
    assert gpu.split_loses(variant, N, M, GZ, K, gpu.Cuda.multiProcessorCount(0)) == 1
    gpu.split_policy(-1)
    rng = np.random.default_rng(N + GZ + variant)
    for dist in ("int", "uniform"):
        A, B = logical_operands(variant, rng, N, M, K, dist=dist)
        before = gpu.declined_splits()
        C, Cbuf = run_sk(gpu, variant, A, B, GZ, summary=False)
        assert gpu.declined_splits() == before + 1
        assert not Cbuf.view(np.uint32).any(), "the partial buffers of a declined split hold exact zeros"
        unsplit, _ = gpu_matmul_2d(gpu, variant, A, B)
        assert np.array_equal(C.view(np.uint32), unsplit.view(np.uint32))
        folded, _ = run_sk(gpu, variant, A, B, GZ, summary=True)
        assert np.array_equal(folded.view(np.uint32), C.view(np.uint32))
        R = oracle.matmul(variant, A, B)
        if dist == "int":
            assert np.array_equal(C, R)
        else:
            assert_within_tolerance(C, R, K, A, B, "%s declined GZ=%d" % (VARIANT_NAMES[variant], GZ))
        # the same call with the slices forced: C + the partials is the same product
        gpu.split_policy(0)
        C0, Cb0 = run_sk(gpu, variant, A, B, GZ, summary=False)
        gpu.split_policy(-1)
        total = C0.astype(np.float64) + Cb0.astype(np.float64).sum(axis=0)
        assert_within_tolerance(total, R, K, A, B, "%s honoured GZ=%d" % (VARIANT_NAMES[variant], GZ))


@pytest.mark.parametrize("variant", [NN, T1, T2])
@pytest.mark.parametrize("shape_gz", [((8, 4096, 4096), 16), ((4100, 8, 2052), 8), ((8, 1000, 1028), 4), ((3000, 4, 516), 3),
                                      ((16, 8192, 1028), 4), ((8200, 32, 516), 2), ((9000, 8, 260), 2)])
def test_the_split_of_a_skinny_product_is_declined(gpu, variant, shape_gz):
    """The host's policy splits the skinny products with few lines (8 x 4096 x 4096: GridZ 16).  The skinny kernel
    cuts K among its workgroups itself: the whole product goes to C through it -- the bits of the unsplit entry
    point --, the partial buffers get exact zeros from the same launch, the fold leaves C as it is; with the
    slices forced the same product comes out of C plus the partials."""
    (N, M, K), GZ = shape_gz
    gpu.split_policy(-1)
    rng = np.random.default_rng(N + M + GZ + variant)
    for dist in ("int", "uniform"):
        A, B = logical_operands(variant, rng, N, M, K, dist=dist)
        before = gpu.declined_splits()
        C, Cbuf = run_sk(gpu, variant, A, B, GZ, summary=False)
        assert gpu.declined_splits() == before + 1
        assert not Cbuf.view(np.uint32).any(), "the partial buffers of a declined split hold exact zeros"
        unsplit, _ = gpu_matmul_2d(gpu, variant, A, B)
        assert np.array_equal(C.view(np.uint32), unsplit.view(np.uint32))
        skipped = gpu.folds_skipped()
        folded, _ = run_sk(gpu, variant, A, B, GZ, summary=True)
        assert gpu.folds_skipped() == skipped + 1
        assert np.array_equal(folded.view(np.uint32), C.view(np.uint32))
        R = oracle.matmul(variant, A, B)
        if dist == "int":
            assert np.array_equal(C, R)
        else:
            assert_within_tolerance(C, R, K, A, B, "%s skinny declined GZ=%d" % (VARIANT_NAMES[variant], GZ))
        gpu.split_policy(0)
        C0, Cb0 = run_sk(gpu, variant, A, B, GZ, summary=False)
        gpu.split_policy(-1)
        total = C0.astype(np.float64) + Cb0.astype(np.float64).sum(axis=0)
        assert_within_tolerance(total, R, K, A, B, "%s skinny honoured GZ=%d" % (VARIANT_NAMES[variant], GZ))


@pytest.mark.parametrize("variant", [NN, T1, T2])
def test_a_winning_split_is_honoured(gpu, variant):
    """256 x 256 x 8192 in 32 slices: 512 (slice, tile) pairs deal whole to the units, the unsplit product has
    sixteen workgroups per tile to put together -- the slices stay, bit for bit where the oracle puts them."""
    (N, M, K), GZ = (256, 256, 8192), 32
    assert gpu.split_loses(variant, N, M, GZ, K, gpu.Cuda.multiProcessorCount(0)) == 0
    gpu.split_policy(-1)
    rng = np.random.default_rng(17 + variant)
    A, B = logical_operands(variant, rng, N, M, K, dist="int")
    before = gpu.declined_splits()
    C, Cbuf = run_sk(gpu, variant, A, B, GZ, summary=False)
    assert gpu.declined_splits() == before
    C0, Cb0 = oracle.matMulSK(variant, GZ, A, B)
    assert np.array_equal(C, C0) and np.array_equal(Cbuf, Cb0)


def test_a_forced_decline_and_a_bias_row(gpu):
    """Policy 1 declines wherever the unsplit product can take the balanced kernel, whatever the estimate
    says; shapes it cannot take (too few stages) keep their slices."""
    gpu.split_policy(1)
    rng = np.random.default_rng(2)
    A, B = logical_operands(T1, rng, 256, 256, 8192, dist="int")
    C, Cbuf = run_sk(gpu, T1, A, B, 32, summary=False)
    assert not Cbuf.view(np.uint32).any() and np.array_equal(C, oracle.matmul(T1, A, B))
    A, B = logical_operands(NN, rng, 64, 64, 256, dist="int")
    C, Cbuf = run_sk(gpu, NN, A, B, 2, summary=False)
    C0, Cb0 = oracle.matMulSK(NN, 2, A, B)
    assert np.array_equal(C, C0) and np.array_equal(Cbuf, Cb0)


def test_the_fold_after_a_declined_split_is_elided_only_when_it_is_a_no_op(gpu):
    """SKbuf_summary with the stream, Cbuf, C, part and sizeC of the declined call just before returns without
    a launch; any other fold, and the same fold after the library has seen a write to C or Cbuf, runs."""
    MM, Cuda = gpu.Cuda_matMul, gpu.Cuda
    N, M, K, GZ = 1000, 780, 1532, 2
    rng = np.random.default_rng(31)
    A, B = logical_operands(NN, rng, N, M, K, dist="int")
    R = oracle.matmul(NN, A, B)
    dA, dB = gpu.DeviceArray(A), gpu.DeviceArray(B)
    dC, dCbuf = gpu.DeviceArray(size=N * M), gpu.DeviceArray(size=N * M)
    s1, s2 = Cuda.newStream_NonBlocking(), Cuda.newStream_NonBlocking()
    gpu.split_policy(-1)

    def declined_call():
        before = gpu.declined_splits()
        MM.matMulSK([s1], 1, GZ, dA.address, dB.address, dC.address, dCbuf.address, N, M, K)
        assert gpu.declined_splits() == before + 1

    # 1. the reference's sequence: elided, C is the product
    declined_call()
    n0 = gpu.folds_skipped()
    MM.SKbuf_summary(s1, dCbuf.address, dC.address, GZ - 1, N * M)
    assert gpu.folds_skipped() == n0 + 1
    Cuda.streamSynchronize(s1)
    assert np.array_equal(dC.get((N, M)), R)
    # 2. the same fold once more: the memory was used up, the kernel runs (adds the zeros in Cbuf)
    MM.SKbuf_summary(s1, dCbuf.address, dC.address, GZ - 1, N * M)
    assert gpu.folds_skipped() == n0 + 1
    Cuda.streamSynchronize(s1)
    assert np.array_equal(dC.get((N, M)), R)
    # 3. the host overwrites Cbuf through the library between the two calls: the fold must add what is there now
    declined_call()
    Cuda.streamSynchronize(s1)
    ones = np.ones(N * M, np.float32)
    Cuda.set1D(s1, dCbuf.address, ones, N * M)
    MM.SKbuf_summary(s1, dCbuf.address, dC.address, GZ - 1, N * M)
    assert gpu.folds_skipped() == n0 + 1
    Cuda.streamSynchronize(s1)
    assert np.array_equal(dC.get((N, M)), R + 1.0)
    # 4. other arguments (another stream; another part): the kernel runs
    declined_call()
    Cuda.streamSynchronize(s1)
    MM.SKbuf_summary(s2, dCbuf.address, dC.address, GZ - 1, N * M)
    assert gpu.folds_skipped() == n0 + 1
    Cuda.streamSynchronize(s2)
    assert np.array_equal(dC.get((N, M)), R)
    # 5. C written by another product of the library in between: the entry is gone, the fold runs on what C holds
    declined_call()
    MM.matMul([s1], 1, dA.address, dB.address, dC.address, N, M, K)
    MM.SKbuf_summary(s1, dCbuf.address, dC.address, GZ - 1, N * M)
    assert gpu.folds_skipped() == n0 + 1
    # 6. switched off: every fold is launched
    gpu.fold_skip(0)
    try:
        declined_call()
        MM.SKbuf_summary(s1, dCbuf.address, dC.address, GZ - 1, N * M)
        assert gpu.folds_skipped() == n0 + 1
        Cuda.streamSynchronize(s1)
        assert np.array_equal(dC.get((N, M)), R)
    finally:
        gpu.fold_skip(1)
    # 7. freed memory takes its entry along: a new allocation at the same address is not mistaken for it
    declined_call()
    Cuda.streamSynchronize(s1)
    address = dCbuf.address
    dCbuf.free()
    dCbuf = gpu.DeviceArray(np.full(N * M, 2.0, np.float32))
    MM.SKbuf_summary(s1, dCbuf.address, dC.address, GZ - 1, N * M)
    assert gpu.folds_skipped() == n0 + 1
    Cuda.streamSynchronize(s1)
    assert np.array_equal(dC.get((N, M)), R + 2.0), "reused address %x / %x" % (address, dCbuf.address)
    for x in (dA, dB, dC, dCbuf):
        x.free()
    Cuda.deleteStream(s1)
    Cuda.deleteStream(s2)
