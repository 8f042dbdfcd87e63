"""Forward convolution as an implicit GEMM on the GPU, through the C ABI, against the CPU oracle
(the reference's naive loops with an FP64 accumulator).  Tolerances as for the products, with
K = FH*FW*IC: relative Frobenius error <= 1e-5, per-element |err| <= 1e-4*sqrt(K)*max|X|*max|W|;
integer-valued inputs must match bit for bit (every summation order is exact there); and the
reference's own acceptance rule (samePercent_relative at 1e-5 >= 0.999 on uniform [0,1) inputs,
test/cuda/conv3D/Cuda_conv3D_test.java:61-93) is evaluated as well."""
import numpy as np
import pytest

from oracle import oracle
from helpers import assert_within_tolerance

pytestmark = pytest.mark.gpu


def pad_last(x, first_to4=False):
    s = (x.shape[-1] + 3) // 4 * 4
    n0 = (x.shape[0] + 3) // 4 * 4 if first_to4 else x.shape[0]
    out = np.zeros((n0,) + x.shape[1:-1] + (s,), np.float32)
    out[:x.shape[0], ..., :x.shape[-1]] = x
    return out


def run_conv(dh, X, W, sh, sw, ph, pw, entry="conv3D", bias=None, fill=7.0):
    """Logical X[N,IH,IW,IC], W[OC,FH,FW,IC] -> logical Y plus the full padded device array."""
    CV = dh.Cuda_conv3D
    N, IH, IW, IC = X.shape
    OC, FH, FW, _ = W.shape
    OH, OW = (IH - FH + 2 * ph) // sh + 1, (IW - FW + 2 * pw) // sw + 1
    Xp, Wp = pad_last(X, first_to4=True), pad_last(W, first_to4=True)    # the engine pads N, IC, OC to x4
    Wp = Wp[:(OC + 3) // 4 * 4]
    N4, IC4, OC4 = Xp.shape[0], Xp.shape[-1], Wp.shape[0]
    dX, dW = dh.DeviceArray(Xp), dh.DeviceArray(Wp)
    dY = dh.DeviceArray(size=N4 * OH * OW * OC4 + 16)
    dY.fill(fill)
    s = [0]
    if entry == "conv3D":
        CV.conv3D(s, 1, dX.address, IH, IW, dW.address, FH, FW, dY.address, OH, OW, N4, IC4, OC4, sh, sw, ph, pw)
    elif entry == "texture":
        CV.conv3D_texture(s, 1, dX.address, IH, IW, dW.address, FH, FW, dY.address, OH, OW, N4, IC4, OC4, sh, sw, ph, pw)
    elif entry == "V2":
        CV.conv3DV2(True, s, 1, dX.address, IH, IW, dW.address, FH, FW, dY.address, OH, OW, N4, IC4, OC4, sh, sw, ph, pw)
    elif entry == "np":
        assert ph == 0 and pw == 0
        CV.conv3D_np(s, 1, dX.address, IH, IW, dW.address, FH, FW, dY.address, OH, OW, N4, IC4, OC4, sh, sw)
    elif entry == "W1":
        assert FH == 1 and FW == 1 and sh == 1 and sw == 1 and ph == 0 and pw == 0
        CV.conv3D_W1(s, 1, dX.address, IH, IW, dW.address, dY.address, N4, IC4, OC4)
    elif entry in ("GemmR", "GemmR_W1", "winograd"):
        dCW = dh.DeviceArray(size=Wp.size)
        CV.kernel_remode(0, dW.address, dCW.address, FH, FW, OC4, IC4)
        if entry == "GemmR":
            CV.conv3D_GemmR(s, 1, dX.address, IH, IW, dW.address, dCW.address, FH, FW, dY.address, OH, OW, N4, IC4,
                            OC4, sh, sw, ph, pw)
        elif entry == "GemmR_W1":
            CV.conv3D_GemmR_W1(s, 1, dX.address, IH, IW, dW.address, dCW.address, dY.address, N4, IC4, OC4)
        else:
            assert sh == 1 and sw == 1
            assert CV.conv3D_Im2col_Winograd_s8_R_texture(True, s, 1, dX.address, IH, IW, dW.address, dCW.address,
                                                          FH, FW, dY.address, OH, OW, N4, IC4, OC4, ph, pw)
        dh.Cuda.streamSynchronize(0)
        CW = dCW.get((FH, FW, IC4, OC4))
        assert np.array_equal(CW, np.transpose(Wp.reshape(OC4, FH, FW, IC4), (1, 2, 3, 0)))   # the re-ordered filter
        dCW.free()
    elif entry == "biased":
        bp = np.zeros(OC4, np.float32); bp[:OC] = bias
        db = dh.DeviceArray(bp)
        CV.conv3D_biased(s, 1, dX.address, IH, IW, dW.address, FH, FW, dY.address, OH, OW, N4, IC4, OC4, sh, sw, ph,
                         pw, db.address, N * OH * OW * OC4, OC)
        dh.Cuda.streamSynchronize(0)
        db.free()
    else:
        raise ValueError(entry)
    dh.Cuda.streamSynchronize(0)
    raw = dY.get()
    for d in (dX, dW, dY):
        d.free()
    assert np.all(raw[N4 * OH * OW * OC4:] == fill)                 # nothing written past Y
    Yp = raw[:N4 * OH * OW * OC4].reshape(N4, OH, OW, OC4)
    return Yp[:N, :, :, :OC], Yp


# IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw: the shapes of the reference's test sweep in small, ragged
# channel counts, strides, paddings up to FH-1, windows hanging over the border, 1x1, tall filters
GEOMS = [(5, 5, 3, 3, 2, 3, 5, 1, 1, 1, 1), (8, 7, 3, 3, 3, 4, 8, 2, 2, 1, 1), (33, 33, 4, 4, 4, 16, 33, 1, 1, 1, 1),
         (32, 32, 3, 3, 4, 16, 64, 2, 2, 1, 1), (6, 6, 1, 1, 5, 7, 9, 1, 1, 0, 0), (7, 9, 3, 2, 2, 5, 6, 2, 1, 0, 0),
         (4, 4, 4, 4, 1, 2, 3, 1, 1, 3, 3), (10, 6, 5, 3, 2, 8, 130, 3, 2, 2, 1), (16, 16, 3, 3, 8, 64, 128, 1, 1, 1, 1),
         (12, 12, 7, 7, 2, 3, 20, 2, 2, 3, 3), (1, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0), (9, 5, 2, 5, 3, 130, 4, 1, 1, 1, 2)]


@pytest.mark.parametrize("geom", GEOMS)
def test_conv3D_matches_oracle(dh, gpu, geom):
    IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw = geom
    rng = np.random.default_rng(sum(geom))
    X = rng.uniform(-1, 1, (N, IH, IW, IC)).astype(np.float32)
    W = rng.uniform(-1, 1, (OC, FH, FW, IC)).astype(np.float32)
    Y, Yp = run_conv(dh, X, W, sh, sw, ph, pw)
    R = oracle.conv3D(X, W, sh, sw, ph, pw)
    assert Y.shape == R.shape
    assert_within_tolerance(Y, R, FH * FW * IC, X, W, "conv3D %s" % (geom,))
    # the reference's rule on the reference's kind of input (random_float_vector: uniform in [0, 1), no cancellation)
    Xq, Wq = rng.random(X.shape, np.float32), rng.random(W.shape, np.float32)
    Yq, _ = run_conv(dh, Xq, Wq, sh, sw, ph, pw)
    assert oracle.samePercent_relative(oracle.conv3D(Xq, Wq, sh, sw, ph, pw), Yq, 1e-5) >= 0.999
    assert not Yp[N:].any() and not Yp[..., OC:].any()              # pad images and pad channels are zeros
    # integer-valued inputs: bit for bit
    Xi = rng.integers(-3, 4, X.shape).astype(np.float32)
    Wi = rng.integers(-3, 4, W.shape).astype(np.float32)
    Yi, _ = run_conv(dh, Xi, Wi, sh, sw, ph, pw)
    assert np.array_equal(Yi, oracle.conv3D(Xi, Wi, sh, sw, ph, pw))


@pytest.mark.parametrize("tile", list(range(-1, 24)) + list(range(256, 266)))
def test_conv3D_every_tile_shape(dh, gpu, tile):
    rng = np.random.default_rng(300 + tile)
    X = rng.integers(-3, 4, (3, 11, 9, 12)).astype(np.float32)
    W = rng.integers(-3, 4, (70, 3, 3, 12)).astype(np.float32)
    dh.force_tile(tile)
    try:
        Y, _ = run_conv(dh, X, W, 2, 1, 1, 1)
    finally:
        dh.force_tile(-1)
    assert np.array_equal(Y, oracle.conv3D(X, W, 2, 1, 1, 1))


@pytest.mark.parametrize("tile", list(range(-1, 15)) + list(range(256, 266)))
def test_conv3D_every_tile_shape_with_whole_channel_stages(dh, gpu, tile):
    # 128 channels: every stage depth (16 ... 128 k) divides them, so every shape takes the loader that keeps
    # the filter tap in scalar registers and visits the filter columns fastest
    rng = np.random.default_rng(400 + tile)
    X = rng.integers(-3, 4, (2, 9, 8, 128)).astype(np.float32)
    W = rng.integers(-3, 4, (40, 3, 3, 128)).astype(np.float32)
    dh.force_tile(tile)
    try:
        Y, _ = run_conv(dh, X, W, 1, 2, 1, 1)
    finally:
        dh.force_tile(-1)
    assert np.array_equal(Y, oracle.conv3D(X, W, 1, 2, 1, 1))


# IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw with channel counts that are multiples of 32
BALANCED_GEOMS = [(9, 8, 3, 3, 2, 128, 40, 1, 2, 1, 1), (14, 14, 3, 3, 5, 64, 70, 1, 1, 1, 1), (7, 7, 1, 1, 9, 96, 130, 1, 1, 0, 0),
                  (12, 10, 7, 7, 3, 32, 64, 2, 2, 3, 3), (6, 6, 5, 4, 2, 64, 12, 1, 1, 4, 3), (20, 20, 3, 3, 2, 32, 200, 3, 1, 0, 2)]


@pytest.mark.parametrize("tile", [18, 19, 20, 21, 22, 23, 25])
@pytest.mark.parametrize("geom", BALANCED_GEOMS)
def test_conv3D_through_the_balanced_kernel(dh, gpu, tile, geom):
    """The gathered operand staged straight into LDS, a filter tap at a time, by workgroups that share the tiles'
    stages in equal runs (tiles 22 and 23 have no such form and fall back).  Integer inputs: bit for bit; with the
    bias row: equal to the oracle's convolution plus the row."""
    IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw = geom
    rng = np.random.default_rng(sum(geom) + tile)
    X = rng.integers(-3, 4, (N, IH, IW, IC)).astype(np.float32)
    W = rng.integers(-3, 4, (OC, FH, FW, IC)).astype(np.float32)
    bias = rng.integers(-5, 6, OC).astype(np.float32)
    R = oracle.conv3D(X, W, sh, sw, ph, pw)
    dh.force_tile(tile)
    try:
        Y, Yp = run_conv(dh, X, W, sh, sw, ph, pw)
        Yb, _ = run_conv(dh, X, W, sh, sw, ph, pw, entry="biased", bias=bias)
    finally:
        dh.force_tile(-1)
    assert np.array_equal(Y, R)
    assert not Yp[N:].any() and not Yp[..., OC:].any()
    assert np.array_equal(Yb, R + bias[None, None, None, :])


@pytest.mark.parametrize("tile", [257, 260, 1])
def test_conv3D_paired_stages_across_tile_boundaries(dh, gpu, tile):
    # more tiles than resident workgroups and nine 16-k stages: a workgroup's second tile starts on the odd
    # LDS buffer, with the filter-tap walk restarted (tile 1: the plain form on the same shape)
    rng = np.random.default_rng(500 + tile)
    X = rng.integers(-3, 4, (48, 64, 64, 16)).astype(np.float32)
    W = rng.integers(-3, 4, (64, 3, 3, 16)).astype(np.float32)
    dh.force_tile(tile)
    try:
        Y, _ = run_conv(dh, X, W, 1, 1, 1, 1)
    finally:
        dh.force_tile(-1)
    assert np.array_equal(Y, oracle.conv3D(X, W, 1, 1, 1, 1))


@pytest.mark.parametrize("entry", ["texture", "V2", "np", "W1", "GemmR", "GemmR_W1", "winograd"])
def test_every_native_family_computes_the_same_convolution(dh, gpu, entry):
    rng = np.random.default_rng(len(entry))
    if entry in ("W1", "GemmR_W1"):
        g = (9, 7, 1, 1, 3, 10, 21, 1, 1, 0, 0)
    elif entry == "np":
        g = (11, 9, 3, 4, 3, 6, 21, 2, 1, 0, 0)
    elif entry == "winograd":
        g = (12, 10, 3, 3, 3, 8, 40, 1, 1, 1, 1)
    else:
        g = (12, 10, 3, 5, 3, 6, 40, 2, 2, 1, 2)
    IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw = g
    X = rng.integers(-3, 4, (N, IH, IW, IC)).astype(np.float32)
    W = rng.integers(-3, 4, (OC, FH, FW, IC)).astype(np.float32)
    Y, _ = run_conv(dh, X, W, sh, sw, ph, pw, entry=entry)
    assert np.array_equal(Y, oracle.conv3D(X, W, sh, sw, ph, pw))


def test_conv3D_at_the_reference_speed_test_shape(dh, gpu):
    # 64 images of 64x64, 64 -> 64 channels, 7x7, padding 3 (test/cuda/conv3D/Cuda_conv3D_test.java main):
    # too large for the CPU loops, so (a) a one-hot filter must copy a shifted channel bit for bit, and
    # (b) 4000 randomly chosen outputs are recomputed in FP64 from their 3136-term definition
    rng = np.random.default_rng(7)
    N, IH, IW, IC, OC, F, P = 64, 64, 64, 64, 64, 7, 3
    X = rng.uniform(-1, 1, (N, IH, IW, IC)).astype(np.float32)
    W = np.zeros((OC, F, F, IC), np.float32)
    for oc in range(OC):
        W[oc, oc % F, (oc // F) % F, (oc * 5) % IC] = 1.0
    Y, _ = run_conv(dh, X, W, 1, 1, P, P)
    Xp = np.zeros((N, IH + 2 * P, IW + 2 * P, IC), np.float32)
    Xp[:, P:P + IH, P:P + IW] = X
    for oc in (0, 1, 13, 48, 63):
        fh, fw, ic = oc % F, (oc // F) % F, (oc * 5) % IC
        assert np.array_equal(Y[..., oc], Xp[:, fh:fh + IH, fw:fw + IW, ic]), oc
    W = rng.uniform(-1, 1, (OC, F, F, IC)).astype(np.float32)
    Y, _ = run_conv(dh, X, W, 1, 1, P, P)
    idx = np.stack([rng.integers(0, N, 4000), rng.integers(0, IH, 4000), rng.integers(0, IW, 4000),
                    rng.integers(0, OC, 4000)], 1)
    Xd, Wd = Xp.astype(np.float64), W.astype(np.float64)
    ref = np.array([np.vdot(Xd[n, oh:oh + F, ow:ow + F, :], Wd[oc]) for n, oh, ow, oc in idx])
    got = Y[idx[:, 0], idx[:, 1], idx[:, 2], idx[:, 3]]
    assert np.abs(got - ref).max() <= 1e-4 * np.sqrt(F * F * IC)
    assert np.linalg.norm(got - ref) <= 1e-5 * np.linalg.norm(ref)


@pytest.mark.parametrize("shape", [(6, 6, 5, 7, 9), (16, 16, 8, 64, 128), (32, 32, 4, 256, 256), (9, 13, 3, 130, 36), (1, 1, 1, 1, 1)])
def test_conv3D_1x1_takes_the_plain_product(dh, gpu, shape):
    """A 1 x 1 filter at stride 1 without padding is the product X[N*IH*IW][IC] * W[OC][IC]^T and is sent to the
    A * B^T kernels, with the bias row in their epilogue: bit for bit on integers, the biased form equal to the
    plain one plus the row, the W1 entry points the same bits; with padding or a stride the gathering loader stays."""
    IH, IW, N, IC, OC = shape
    rng = np.random.default_rng(sum(shape))
    X = rng.integers(-3, 4, (N, IH, IW, IC)).astype(np.float32)
    W = rng.integers(-3, 4, (OC, 1, 1, IC)).astype(np.float32)
    bias = rng.integers(-5, 6, OC).astype(np.float32)
    R = oracle.conv3D(X, W, 1, 1, 0, 0)
    Y, Yp = run_conv(dh, X, W, 1, 1, 0, 0)
    assert np.array_equal(Y, R)
    assert not Yp[N:].any() and not Yp[..., OC:].any()
    Yb, Ybp = run_conv(dh, X, W, 1, 1, 0, 0, entry="biased", bias=bias)
    assert np.array_equal(Yb, R + bias[None, None, None, :])
    assert not Ybp[N:].any() and not Ybp[..., OC:].any()
    Yw, _ = run_conv(dh, X, W, 1, 1, 0, 0, entry="W1")
    assert np.array_equal(Yw, R)
    Xu = rng.uniform(-1, 1, X.shape).astype(np.float32)
    Wu = rng.uniform(-1, 1, W.shape).astype(np.float32)
    Yu, _ = run_conv(dh, Xu, Wu, 1, 1, 0, 0)
    ref = oracle.conv3D(Xu, Wu, 1, 1, 0, 0)
    assert np.abs(Yu - ref).max() <= 1e-4 * np.sqrt(IC) and np.linalg.norm(Yu - ref) <= 1e-5 * np.linalg.norm(ref) + 1e-30
    Ys, _ = run_conv(dh, X, W, 2, 1, 0, 0)
    assert np.array_equal(Ys, oracle.conv3D(X, W, 2, 1, 0, 0))


def test_conv3D_biased_equals_two_launches(dh, gpu):
    rng = np.random.default_rng(9)
    X = rng.uniform(-1, 1, (3, 10, 9, 7)).astype(np.float32)
    W = rng.uniform(-1, 1, (37, 3, 3, 7)).astype(np.float32)
    bias = rng.uniform(-2, 2, 37).astype(np.float32)
    Yb, Ypb = run_conv(dh, X, W, 1, 2, 1, 1, entry="biased", bias=bias)
    Y, _ = run_conv(dh, X, W, 1, 2, 1, 1)
    assert np.array_equal(Yb.view(np.uint32), ((Y + bias) + np.float32(0)).view(np.uint32))   # an exact float add
    assert not Ypb[3:].any() and not Ypb[..., 37:].any()


def test_conv3D_argument_errors(dh, gpu):
    CV = dh.Cuda_conv3D
    d = dh.DeviceArray(size=4096)
    a = d.address
    ok = dict(dX=a, IH=4, IW=4, dW=a + 2048, FH=3, FW=3, dY=a + 8192, OH=4, OW=4, N=4, IC=4, OC=4, sh=1, sw=1, ph=1, pw=1)

    def call(**kw):
        g = dict(ok); g.update(kw)
        CV.conv3D([0], 1, g["dX"], g["IH"], g["IW"], g["dW"], g["FH"], g["FW"], g["dY"], g["OH"], g["OW"], g["N"],
                  g["IC"], g["OC"], g["sh"], g["sw"], g["ph"], g["pw"])
    call()
    for bad in (dict(dX=0), dict(dW=0), dict(dY=0), dict(IC=3), dict(OC=6), dict(sh=0), dict(ph=-1), dict(FH=0),
                dict(OH=0), dict(N=0), dict(dX=a + 4), dict(IC=1 << 22, FH=3, FW=3)):
        with pytest.raises(dh.CudaException) as e:
            call(**bad)
        assert e.value.code == 1, bad
    dh.Cuda.streamSynchronize(0)
    d.free()


# ---- engine level -----------------------------------------------------------------------------------

@pytest.fixture(scope="module", params=["direct", "pooled"])
def eg(gpu, request):
    """With and without the recycling device memory pool behind the tensors (recycled blocks are dirty)."""
    from dragon_hip import engine
    e = engine.cuda_float32(0, 32, max_mem_size=(2 << 30) if request.param == "pooled" else 0)
    yield e
    e.close()


def check_conv(eg, rng, IH, IW, FH, FW, N, IC, OC, sh, sw, ph, pw):
    """testCorrect of test/cuda/conv3D/Cuda_conv3D_test.java:42-105: both forms of eg.conv3D against the
    CPU loops by samePercent_relative at 1e-5, plus conv3D_biased == conv3D then add_row, exactly."""
    OH, OW = (IH - FH + 2 * ph) // sh + 1, (IW - FW + 2 * pw) // sw + 1
    X = rng.random(N * IH * IW * IC, dtype=np.float32)
    W = rng.random(OC * FH * FW * IC, dtype=np.float32)
    Bv = rng.random(OC, dtype=np.float32)
    tX, tW, tB = eg.tensor(X, N, IH, IW, IC), eg.tensor(W, OC, FH, FW, IC), eg.tensor(Bv, OC)
    tY1 = eg.conv3D(tX, tW, sh, sw, ph, pw)
    tY2 = eg.conv3D(eg.empty(N, OH, OW, OC).c(), tX, tW, sh, sw)
    assert tY1.dim == [N, OH, OW, OC]
    Y1 = oracle.conv3D(X.reshape(N, IH, IW, IC), W.reshape(OC, FH, FW, IC), sh, sw, ph, pw).reshape(-1)
    Y2, Y3 = eg.valueOf(tY1), eg.valueOf(tY2)
    assert oracle.samePercent_relative(Y1, Y2, 1e-5) >= 0.999
    if ((OH - 1) * sh + FH - IH + 1) >> 1 == ph and ((OW - 1) * sw + FW - IW + 1) >> 1 == pw:
        assert np.array_equal(Y2, Y3)                          # the derived padding is the one given
    tY4 = eg.conv3D_biased(tX, tW, sh, sw, ph, pw, tB)
    tY5 = eg.add_row(True, eg.conv3D(tX, tW, OH, OW, sh, sw, ph, pw), tB)
    assert np.array_equal(eg.valueOf(tY4), eg.valueOf(tY5))
    tY6 = eg.conv3D_biased(eg.zeros(N, OH, OW, OC).c(), tX, tW, sh, sw, ph, pw, tB)
    assert np.array_equal(eg.valueOf(tY4), eg.valueOf(tY6))
    # pads of Y stay zero: images beyond N, channels beyond OC
    from dragon_hip import Cuda
    raw = np.empty(tY4.length_4x, np.float32)
    Cuda.get1D(0, tY4.address, raw, tY4.length_4x)
    raw = raw.reshape((N + 3) // 4 * 4, OH, OW, (OC + 3) // 4 * 4)
    assert not raw[N:].any() and not raw[..., OC:].any()
    eg.delete(tX, tW, tB, tY1, tY2, tY4, tY5, tY6)


SHAPES = [(8, 8, 3, 3, 4, 16, 32, 1, 1, 1, 1), (9, 7, 3, 3, 3, 5, 33, 2, 2, 1, 1), (16, 16, 7, 7, 2, 8, 64, 1, 1, 3, 3),
          (12, 12, 1, 1, 5, 128, 37, 1, 1, 0, 0), (33, 33, 5, 5, 4, 16, 19, 2, 2, 0, 0), (6, 10, 1, 7, 2, 6, 40, 1, 1, 0, 3),
          (2, 2, 3, 3, 16, 32, 48, 2, 2, 1, 1)]


@pytest.mark.parametrize("remode,fused", [(0, 1), (1, 1), (0, 0), (1, 0)])
def test_engine_conv3D_like_the_reference(eg, remode, fused):
    rng = np.random.default_rng(40 + 2 * remode + fused)
    base = eg.get_param("live_blocks")
    eg.set_param("conv3D_remode", remode)
    eg.set_param("conv3D_biased_fused", fused)
    try:
        for g in SHAPES:
            check_conv(eg, rng, *g)
    finally:
        eg.set_param("conv3D_remode", 0)
        eg.set_param("conv3D_biased_fused", 1)
    assert eg.get_param("live_blocks") == base                 # the re-ordered filter's block went back


def test_engine_conv3D_async_and_stream_counts(eg):
    rng = np.random.default_rng(50)
    N, IH, IW, IC, OC = 4, 10, 10, 8, 36
    X = rng.integers(-2, 3, (N, IH, IW, IC)).astype(np.float32)
    W = rng.integers(-2, 3, (OC, 3, 3, IC)).astype(np.float32)
    tX, tW = eg.tensor(X, N, IH, IW, IC), eg.tensor(W, OC, 3, 3, IC)
    eg.sync(False)
    try:
        outs = [eg.conv3D(tX, tW, 1, 1, 1, 1) for _ in range(6)]
        assert eg.get_param("last_stream_count") == eg.conv3D_GEMM_nstream(N * IH * IW, OC)
        R = oracle.conv3D(X, W, 1, 1, 1, 1).reshape(-1)
        for t in outs:
            assert np.array_equal(eg.valueOf(t.c()), R)
    finally:
        eg.sync(True)
    eg.delete(tX, tW, *outs)


def test_engine_conv3D_error_behaviour(eg):
    from dragon_hip.engine import IllegalArgumentException, NullPointerException
    tX, tW = eg.zeros(2, 6, 6, 4), eg.zeros(8, 3, 3, 4)
    with pytest.raises(IllegalArgumentException):
        eg.conv3D(tX, eg.zeros(8, 3, 3, 5), 1, 1, 1, 1)        # W.IC != X.IC
    with pytest.raises(IllegalArgumentException):
        eg.conv3D(tX, tW, 1, 1, 3, 1)                          # FH <= ph
    with pytest.raises(IllegalArgumentException):
        eg.conv3D(tX, tW, 4, 1, 1, 1)                          # FH < sh
    with pytest.raises(IllegalArgumentException):
        eg.conv3D(tX, tW, 0, 1, 1, 1)
    with pytest.raises(IllegalArgumentException):
        eg.conv3D(eg.zeros(2, 2, 2, 4), eg.zeros(8, 5, 5, 4), 1, 1, 1, 1)   # FH > IH + 2 ph
    with pytest.raises(IllegalArgumentException):
        eg.conv3D(eg.zeros(2, 6, 6, 7), tX, tW, 1, 1)          # Y.OC != W.OC
    with pytest.raises(IllegalArgumentException):
        eg.conv3D_biased(tX, tW, 1, 1, 1, 1, eg.zeros(9))      # Bias.lastDim != OC
    with pytest.raises(NullPointerException):
        eg.conv3D(None, tW, 1, 1, 1, 1)
    assert eg.conv3D_GEMM_nstream(64, 64) == 1 and eg.conv3D_GEMM_nstream(196, 36) == 6
    assert eg.conv3D_GEMM_nstream(255 * 4, 252) == 10
