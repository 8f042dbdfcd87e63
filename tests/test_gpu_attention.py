"""The attention block in one launch (softmax(scale * Q.K^T).V without the score matrix in memory)
against the reference's operator chain restated on the CPU (oracle.attention: batchMatMulT2, sdiv,
softmax, batchMatMul in float, nn/unit/complex/block/ChannelMHA.java:74-78) and against the same
mathematics in FP64.

Tolerance.  Y is a convex combination of the rows of V, so |Y| <= max|V|; the float chain and the
fused kernel both carry the rounding of the scores (K = d products), of the exponentials and of a
sum over VL terms.  Gate: relative Frobenius error <= 1e-5 and per-element
|err| <= 1e-4 * sqrt(d) * max|V| * (1 + |scale| * max|Q| * max|K|) against FP64 (the second factor is
the sensitivity of the softmax to the rounding of its scores), and the fused result must be at least as
close to FP64 as twice the float chain's own distance plus 1e-6."""
import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu


def pad_last(x):
    s = (x.shape[-1] + 3) // 4 * 4
    out = np.zeros(x.shape[:-1] + (s,), np.float32)
    out[..., :x.shape[-1]] = x
    return out


def attention_f64(Q, K, V, scale):
    """[N, head, L, d] logical arrays."""
    S = np.einsum("nhqd,nhkd->nhqk", Q.astype(np.float64), K.astype(np.float64)) * np.float64(np.float32(scale))
    P = np.exp(S - S.max(-1, keepdims=True))
    P /= P.sum(-1, keepdims=True)
    return np.einsum("nhqk,nhkd->nhqd", P, V.astype(np.float64))


def run_attention(dh, Q, K, V, scale, head_inner, fill=7.0):
    """Q[N, head, QL, dk], K[N, head, VL, dk], V[N, head, VL, dv] logical; returns Y[N, head, QL, dv] and the
    raw padded device array.  With head_inner the device tensors are [N, L, head, d4]."""
    N, H, QL, dk = Q.shape
    VL, dv = V.shape[2], V.shape[3]
    Qp, Kp, Vp = pad_last(Q), pad_last(K), pad_last(V)
    dk4, dv4 = Qp.shape[-1], Vp.shape[-1]
    if head_inner:
        Qp, Kp, Vp = (np.ascontiguousarray(x.transpose(0, 2, 1, 3)) for x in (Qp, Kp, Vp))
    dQ, dK, dV = dh.DeviceArray(Qp), dh.DeviceArray(Kp), dh.DeviceArray(Vp)
    ny = N * H * QL * dv4
    dY = dh.DeviceArray(size=ny + 16)
    dY.fill(fill)
    dh.Cuda_attention.forward([0], 1, dQ.address, dK.address, dV.address, dY.address, N, H, QL, VL, dk4, dv4,
                              head_inner, scale)
    dh.Cuda.streamSynchronize(0)
    raw = dY.get()
    for d in (dQ, dK, dV, dY):
        d.free()
    assert np.all(raw[ny:] == fill)
    Yp = raw[:ny].reshape((N, QL, H, dv4) if head_inner else (N, H, QL, dv4))
    if head_inner:
        Yp = Yp.transpose(0, 2, 1, 3)
    assert not Yp[..., dv:].any()                        # the pad columns of Y are zeros
    return Yp[..., :dv]


def check(dh, rng, N, H, QL, VL, dk, dv, scale, head_inner, amp=1.0):
    Q = rng.uniform(-amp, amp, (N, H, QL, dk)).astype(np.float32)
    K = rng.uniform(-amp, amp, (N, H, VL, dk)).astype(np.float32)
    V = rng.uniform(-1, 1, (N, H, VL, dv)).astype(np.float32)
    Y = run_attention(dh, Q, K, V, scale, head_inner)
    R64 = attention_f64(Q, K, V, scale)
    R32 = oracle.attention(Q.reshape(N * H, QL, dk), K.reshape(N * H, VL, dk), V.reshape(N * H, VL, dv),
                           scale).reshape(N, H, QL, dv)
    assert np.isfinite(Y).all()
    e_dev, e_ref = np.abs(Y - R64).max(), np.abs(R32 - R64).max()
    bound = 1e-4 * np.sqrt(dk) * np.abs(V).max() * (1 + abs(scale) * np.abs(Q).max() * np.abs(K).max())
    assert np.linalg.norm(Y - R64) <= 1e-5 * np.linalg.norm(R64), (N, H, QL, VL, dk, dv)
    assert e_dev <= bound, (e_dev, bound)
    assert e_dev <= 2 * e_ref + 1e-6, (e_dev, e_ref)
    return Y


SHAPES = [  # N, head, QL, VL, dk, dv
    (1, 1, 1, 1, 4, 4), (2, 3, 37, 29, 20, 20), (1, 2, 128, 128, 64, 64), (2, 2, 130, 257, 64, 64),
    (1, 4, 300, 31, 32, 32), (1, 1, 64, 1000, 61, 64), (3, 1, 5, 33, 7, 40), (1, 2, 129, 64, 40, 12),
    (1, 1, 255, 96, 64, 8), (1, 2, 100, 150, 128, 128), (1, 1, 70, 90, 96, 72), (2, 1, 33, 65, 100, 128),
    (1, 1, 129, 40, 16, 125),
    # head dimensions above 128: eight 32-wide blocks per query, one workgroup per compute unit
    (1, 2, 130, 70, 132, 132), (2, 1, 100, 257, 256, 256), (1, 1, 64, 64, 192, 40), (1, 3, 37, 90, 20, 200),
    (1, 1, 200, 130, 192, 192), (1, 2, 66, 200, 160, 160), (1, 1, 129, 65, 224, 224), (1, 1, 129, 130, 80, 80)]


@pytest.mark.parametrize("head_inner", [0, 1])
@pytest.mark.parametrize("shape", SHAPES)
def test_attention_matches_the_chain_and_fp64(dh, gpu, shape, head_inner):
    N, H, QL, VL, dk, dv = shape
    rng = np.random.default_rng(sum(shape) + head_inner)
    check(dh, rng, N, H, QL, VL, dk, dv, 1.0 / np.sqrt(H * dk), head_inner)


def test_attention_scale_variants_and_sharp_rows(dh, gpu):
    rng = np.random.default_rng(77)
    for scale, amp in ((1.0, 1.0), (-0.5, 1.0), (0.0, 1.0), (4.0, 3.0)):
        check(dh, rng, 1, 2, 70, 90, 24, 24, scale, 0, amp)
    # one key dominates: Y equals that key's row of V to float accuracy
    Q = np.zeros((1, 1, 40, 8), np.float32); Q[..., 0] = 50.0
    K = np.zeros((1, 1, 70, 8), np.float32); K[0, 0, 41, 0] = 1.0
    V = rng.uniform(-1, 1, (1, 1, 70, 16)).astype(np.float32)
    Y = run_attention(dh, Q, K, V, 1.0, 0)
    assert np.abs(Y - V[0, 0, 41]).max() <= 1e-6
    # equal scores: Y is the plain mean of V
    Y = run_attention(dh, np.zeros_like(Q), K, V, 1.0, 0)
    assert np.abs(Y - V.astype(np.float64).mean(2)).max() <= 1e-6
    # a value far above the float range of exp stays finite (the maximum is subtracted first)
    Q[..., 0] = 3e4
    K[0, 0, :, 0] = rng.uniform(-3e4, 3e4, 70).astype(np.float32)
    Y = run_attention(dh, Q, K, V, 1.0, 0)
    assert np.isfinite(Y).all() and np.abs(Y - V[0, 0, np.argmax(K[0, 0, :, 0])]).max() <= 1e-6


@pytest.mark.parametrize("step", [0.02, 0.3, 2.0, 9.0, -0.3])
def test_attention_with_scores_that_keep_rising(dh, gpu, step):
    # The kernel lets its reference maximum lag behind the true running maximum (it is raised only when a
    # score exceeds it by 2^8).  Scores that climb a little with every key never trigger the raise for
    # long stretches, scores that climb fast trigger it every step, falling scores never after the first:
    # all must give the FP64 result.
    rng = np.random.default_rng(31)
    VL, d = 700, 16
    Q = np.zeros((1, 1, 70, d), np.float32); Q[..., 0] = 1.0
    Q[0, 0, :, 1] = rng.uniform(-1, 1, 70)
    K = np.zeros((1, 1, VL, d), np.float32)
    K[0, 0, :, 0] = (step * np.arange(VL)).astype(np.float32)
    K[0, 0, :, 1] = rng.uniform(-1, 1, VL)
    V = rng.uniform(-1, 1, (1, 1, VL, d)).astype(np.float32)
    Y = run_attention(dh, Q, K, V, 1.0, 0)
    R = attention_f64(Q, K, V, 1.0)
    assert np.isfinite(Y).all()
    # a score of size |s| carries a rounding error of 2^-24 |s|, which the exponential turns into a relative one
    smax = np.abs(np.einsum("nhqd,nhkd->nhqk", Q.astype(np.float64), K.astype(np.float64))).max()
    assert np.abs(Y - R).max() <= 2e-6 + 2.0 ** -23 * smax, (np.abs(Y - R).max(), smax)
    R32 = oracle.attention(Q[0], K[0], V[0], 1.0)
    assert np.abs(Y - R).max() <= 2 * np.abs(R32 - R[0]).max() + 2e-6       # no worse than the float chain


def test_attention_equals_the_device_chain(dh, gpu):
    # the same block through the three launches it replaces
    rng = np.random.default_rng(5)
    B, QL, VL, d = 8, 200, 168, 64
    Q = rng.standard_normal((1, B, QL, d)).astype(np.float32)
    K = rng.standard_normal((1, B, VL, d)).astype(np.float32)
    V = rng.standard_normal((1, B, VL, d)).astype(np.float32)
    Y = run_attention(dh, Q, K, V, 0.125, 0)
    dQ, dK, dV = dh.DeviceArray(Q), dh.DeviceArray(K), dh.DeviceArray(V)
    dP, dO = dh.DeviceArray(size=B * QL * VL), dh.DeviceArray(size=B * QL * d)
    BMM = dh.Cuda_batchMatMul
    BMM.batchMatMulT2([0], 1, dQ.address, dK.address, dP.address, B, QL, VL, VL, d)
    dh.Cuda_reduce.softmax2D(0, dP.address, dP.address, B * QL, VL, VL, VL, 0.125)
    BMM.batchMatMul([0], 1, dP.address, dV.address, dO.address, B, QL, d, VL, VL)
    dh.Cuda.streamSynchronize(0)
    O = dO.get()[:B * QL * d].reshape(1, B, QL, d)
    for x in (dQ, dK, dV, dP, dO):
        x.free()
    assert np.abs(Y - O).max() <= 2e-6 * max(1.0, np.abs(V).max())


def test_attention_at_the_full_batched_workload_shape(dh, gpu):
    # 4 images x 16 heads, 1024 queries and keys, 64 per head (the shape of the batched benchmark workload):
    # the one-launch block against the three launches it replaces, both layouts, plus two properties that do
    # not depend on the size: rows of V all equal -> Y equals that row; Y lies within the range of V
    rng = np.random.default_rng(64)
    N, H, L, d = 4, 16, 1024, 64
    Q = (rng.standard_normal((N, H, L, d)) * 0.5).astype(np.float32)
    K = (rng.standard_normal((N, H, L, d)) * 0.5).astype(np.float32)
    V = rng.standard_normal((N, H, L, d)).astype(np.float32)
    Y0 = run_attention(dh, Q, K, V, 0.125, 0)
    Y1 = run_attention(dh, Q, K, V, 0.125, 1)
    assert np.array_equal(Y0, Y1)                        # the layout changes addresses, not arithmetic
    dQ, dK, dV = dh.DeviceArray(Q), dh.DeviceArray(K), dh.DeviceArray(V)
    B = N * H
    dP, dO = dh.DeviceArray(size=B * L * L), dh.DeviceArray(size=B * L * d)
    BMM = dh.Cuda_batchMatMul
    BMM.batchMatMulT2([0], 1, dQ.address, dK.address, dP.address, B, L, L, L, d)
    dh.Cuda_reduce.softmax2D(0, dP.address, dP.address, B * L, L, L, L, 0.125)
    BMM.batchMatMul([0], 1, dP.address, dV.address, dO.address, B, L, d, L, L)
    dh.Cuda.streamSynchronize(0)
    O = dO.get().reshape(N, H, L, d)
    for x in (dQ, dK, dV, dP, dO):
        x.free()
    assert np.abs(Y0 - O).max() <= 4e-6 * np.abs(V).max()
    assert np.linalg.norm(Y0 - O) <= 1e-5 * np.linalg.norm(O)
    assert Y0.max() <= V.max() and Y0.min() >= V.min()
    Vc = np.broadcast_to(V[:, :, :1, :], V.shape).copy()
    Yc = run_attention(dh, Q, K, Vc, 0.125, 0)
    assert np.abs(Yc - Vc[:, :, :1, :]).max() <= 2e-6 * np.abs(V).max()


def test_attention_argument_errors(dh, gpu):
    d = dh.DeviceArray(size=65536)
    a = d.address
    ok = dict(dQ=a, dK=a + 4096, dV=a + 8192, dY=a + 16384, N=1, head=2, QL=8, VL=8, dK4=8, dV4=8, hi=0, scale=1.0)

    def call(**kw):
        g = dict(ok); g.update(kw)
        dh.Cuda_attention.forward([0], kw.get("length", 1), g["dQ"], g["dK"], g["dV"], g["dY"], g["N"], g["head"],
                                  g["QL"], g["VL"], g["dK4"], g["dV4"], g["hi"], g["scale"])
    call()
    for bad in (dict(dQ=0), dict(dK=0), dict(dV=0), dict(dY=0), dict(dQ=a + 4), dict(N=0), dict(head=0), dict(QL=0),
                dict(VL=0), dict(dK4=6), dict(dV4=0), dict(dK4=260), dict(dV4=512), dict(scale=float("nan")), dict(scale=float("inf")),
                dict(length=0), dict(length=11)):
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


@pytest.mark.parametrize("shape", [(2, 37, 29, 4, 20, 20), (1, 130, 130, 2, 64, 32), (3, 16, 50, 1, 7, 9),
                                   (2, 64, 64, 8, 8, 8), (1, 140, 70, 2, 128, 96)])
def test_engine_attention_equals_the_block_of_the_reference(eg, shape):
    # ChannelMHA.java:66-83 through the engine mirror, operator by operator, against the one-launch form
    N, QL, VL, head, dk, dv = shape
    rng = np.random.default_rng(sum(shape))
    KC, VC = head * dk, head * dv
    Q = rng.uniform(-1, 1, (N, QL, KC)).astype(np.float32)
    K = rng.uniform(-1, 1, (N, VL, KC)).astype(np.float32)
    V = rng.uniform(-1, 1, (N, VL, VC)).astype(np.float32)
    base = eg.get_param("live_blocks")
    tQ, tK, tV = (eg.tensor(x, *x.shape) for x in (Q, K, V))
    tY = eg.attention(tQ, tK, tV, head)
    assert tY.dim == [N, QL, VC]
    Y = eg.valueOf(tY).reshape(N, QL, head, dv)
    # the chain on [N, L, head, d] views
    t4 = [eg.tensor(x.reshape(N, -1, head, d), N, x.shape[1], head, d) for x, d in ((Q, dk), (K, dk), (V, dv))]
    tQt, tKt, tVt = (eg.transpose(False, t, 1, 2) for t in t4)
    tP = eg.softmax(True, eg.batchMatMulT2(tQt, tKt), scale=float(1 / np.sqrt(KC)))
    tO = eg.transpose(True, eg.batchMatMul(tP, tVt), 1, 2)
    O = eg.valueOf(tO).reshape(N, QL, head, dv)
    assert np.abs(Y - O).max() <= 2e-6
    R = attention_f64(Q.reshape(N, QL, head, dk).transpose(0, 2, 1, 3), K.reshape(N, VL, head, dk).transpose(0, 2, 1, 3),
                      V.reshape(N, VL, head, dv).transpose(0, 2, 1, 3), 1 / np.sqrt(KC)).transpose(0, 2, 1, 3)
    assert np.linalg.norm(Y - R) <= 1e-5 * np.linalg.norm(R)
    eg.delete(tQ, tK, tV, tY, tQt, tKt, tVt, tP, tO, *t4)
    assert eg.get_param("live_blocks") == base


def test_engine_attention_error_behaviour(eg):
    from dragon_hip.engine import IllegalArgumentException, NullPointerException
    tQ, tK, tV = eg.zeros(2, 8, 24), eg.zeros(2, 9, 24), eg.zeros(2, 9, 24)
    with pytest.raises(IllegalArgumentException):
        eg.attention(tQ, tK, tV, 5)                            # seq_dim mod head
    with pytest.raises(IllegalArgumentException):
        eg.attention(tQ, tK, tV, 4)                            # head dimension 6 is no multiple of 4
    with pytest.raises(IllegalArgumentException):
        eg.attention(tQ, eg.zeros(2, 9, 20), tV, 1)            # K.seq_dim != Q.seq_dim
    with pytest.raises(IllegalArgumentException):
        eg.attention(tQ, tK, eg.zeros(2, 10, 24), 1)           # K.seq_len != V.seq_len
    with pytest.raises(IllegalArgumentException):
        eg.attention(eg.zeros(2, 8, 260), eg.zeros(2, 9, 260), tV, 1)   # head dimension above 256
    with pytest.raises(NullPointerException):
        eg.attention(None, tK, tV, 1)
    assert eg.attention(tQ, tK, tV, 2).dim == [2, 8, 24]


# ---- the block's mask: a tensor that multiplies the probabilities after the softmax (ChannelMHA.java:75-76) ----

def attention_masked_f64(Q, K, V, scale, M):
    S = np.einsum("nhqd,nhkd->nhqk", Q.astype(np.float64), K.astype(np.float64)) * np.float64(np.float32(scale))
    P = np.exp(S - S.max(-1, keepdims=True))
    P /= P.sum(-1, keepdims=True)
    return np.einsum("nhqk,nhkd->nhqd", P * M.astype(np.float64), V.astype(np.float64))


def run_attention_masked(dh, Q, K, V, M, scale, head_inner, garbage_pad=False):
    """M[QL, VL] (one mask for every image and head) or M[N, head, QL, VL]."""
    N, H, QL, dk = Q.shape
    VL, dv = V.shape[2], V.shape[3]
    Qp, Kp, Vp, Mp = pad_last(Q), pad_last(K), pad_last(V), pad_last(M)
    if garbage_pad:                                      # nothing beyond the last key may count
        Mp[..., VL:] = np.float32("inf")
    dk4, dv4 = Qp.shape[-1], Vp.shape[-1]
    if head_inner:
        Qp, Kp, Vp = (np.ascontiguousarray(x.transpose(0, 2, 1, 3)) for x in (Qp, Kp, Vp))
    dQ, dK, dV, dM = dh.DeviceArray(Qp), dh.DeviceArray(Kp), dh.DeviceArray(Vp), dh.DeviceArray(Mp)
    ny = N * H * QL * dv4
    dY = dh.DeviceArray(size=ny + 16)
    dY.fill(3.0)
    dh.Cuda_attention.forward_masked([0], 1, dQ.address, dK.address, dV.address, dM.address, dY.address, N, H, QL, VL,
                                     dk4, dv4, head_inner, scale, Mp.shape[-1], M.ndim == 4)
    dh.Cuda.streamSynchronize(0)
    raw = dY.get()
    for d in (dQ, dK, dV, dM, dY):
        d.free()
    assert np.all(raw[ny:] == 3.0)
    Yp = raw[:ny].reshape((N, QL, H, dv4) if head_inner else (N, H, QL, dv4))
    if head_inner:
        Yp = Yp.transpose(0, 2, 1, 3)
    assert not Yp[..., dv:].any()
    return Yp[..., :dv]


MASKED_SHAPES = [(1, 1, 1, 1, 4, 4), (2, 3, 37, 29, 20, 20), (1, 2, 128, 128, 64, 64), (2, 2, 130, 257, 64, 64),
                 (1, 2, 200, 333, 128, 96), (3, 1, 65, 64, 32, 8), (1, 4, 300, 70, 12, 100), (1, 2, 70, 100, 160, 256),
                 # three, five, six and seven of the tile row's 32-wide blocks in use
                 (1, 2, 50, 80, 72, 96), (1, 1, 40, 64, 160, 132), (1, 2, 70, 100, 192, 160), (1, 1, 40, 64, 36, 224)]


@pytest.mark.parametrize("head_inner", [False, True])
@pytest.mark.parametrize("kind", ["causal", "dropout", "signed", "per head"])
def test_masked_block_against_the_chain_and_fp64(dh, gpu, head_inner, kind):
    rng = np.random.default_rng(515 + len(kind) + 7 * head_inner)
    for (N, H, QL, VL, dk, dv) in MASKED_SHAPES:
        Q = rng.uniform(-1, 1, (N, H, QL, dk)).astype(np.float32)
        K = rng.uniform(-1, 1, (N, H, VL, dk)).astype(np.float32)
        V = rng.uniform(-1, 1, (N, H, VL, dv)).astype(np.float32)
        if kind == "causal":
            M = (np.arange(VL)[None, :] <= np.arange(QL)[:, None] * VL // QL).astype(np.float32)
        elif kind == "dropout":
            M = (rng.uniform(0, 1, (QL, VL)) >= 0.3).astype(np.float32) / np.float32(0.7)
        elif kind == "signed":
            M = rng.uniform(-2, 2, (QL, VL)).astype(np.float32)
        else:
            M = rng.uniform(0, 1.5, (N, H, QL, VL)).astype(np.float32)
        scale = 1.0 / np.sqrt(dk)
        Y = run_attention_masked(dh, Q, K, V, M, scale, head_inner, garbage_pad=(kind == "signed"))
        M4 = np.broadcast_to(M, (N, H, QL, VL))
        R64 = attention_masked_f64(Q, K, V, scale, M4)
        R32 = oracle.attention(Q.reshape(N * H, QL, dk), K.reshape(N * H, VL, dk), V.reshape(N * H, VL, dv), scale,
                               mask=M4.reshape(N * H, QL, VL)).reshape(N, H, QL, dv)
        assert np.isfinite(Y).all()
        e_dev, e_ref = np.abs(Y - R64).max(), np.abs(R32 - R64).max()
        bound = 1e-4 * np.sqrt(dk) * np.abs(V).max() * np.abs(M).max() * (1 + abs(scale) * np.abs(Q).max() * np.abs(K).max())
        assert np.linalg.norm(Y - R64) <= 1e-5 * max(np.linalg.norm(R64), 1e-30) + 1e-7, (kind, N, H, QL, VL, dk, dv)
        assert e_dev <= bound and e_dev <= 2 * e_ref + 1e-6, (kind, e_dev, e_ref, bound)


def test_masked_block_exact_cases(dh, gpu):
    rng = np.random.default_rng(77)
    N, H, QL, VL, d = 1, 2, 70, 90, 16
    Q = rng.uniform(-1, 1, (N, H, QL, d)).astype(np.float32)
    K = rng.uniform(-1, 1, (N, H, VL, d)).astype(np.float32)
    V = rng.uniform(-1, 1, (N, H, VL, d)).astype(np.float32)
    # a mask of ones is no mask: the same bits as the unmasked entry point
    Y1 = run_attention_masked(dh, Q, K, V, np.ones((QL, VL), np.float32), 0.25, False)
    Y0 = run_attention(dh, Q, K, V, 0.25, False)
    assert np.array_equal(Y1, Y0)
    # a mask of zeros gives zeros; a mask that keeps one key gives that key's row of V times its probability
    assert not run_attention_masked(dh, Q, K, V, np.zeros((QL, VL), np.float32), 0.25, False).any()
    M = np.zeros((QL, VL), np.float32)
    M[:, 5] = 1.0
    Y = run_attention_masked(dh, Q * 0, K, V, M, 0.25, False)          # equal scores: probability 1 / VL
    assert np.allclose(Y, V[:, :, 5:6, :] / VL, rtol=1e-6, atol=1e-7)


def test_masked_block_argument_errors(dh, gpu):
    d = dh.DeviceArray(size=4096)
    a = d.address
    f = dh.Cuda_attention.forward_masked
    with pytest.raises(dh.CudaException):
        f([0], 1, a, a, a, 0, a, 1, 1, 8, 8, 4, 4, False, 1.0, 8, False)        # no mask
    with pytest.raises(dh.CudaException):
        f([0], 1, a, a, a, a, a, 1, 1, 8, 8, 4, 4, False, 1.0, 4, False)        # pitch below the key count
    with pytest.raises(dh.CudaException):
        f([0], 1, a, a, a, a, a, 1, 1, 8, 6, 4, 4, False, 1.0, 6, False)        # pitch not a multiple of 4
    with pytest.raises(dh.CudaException):
        f([0], 1, a, a, a, a + 4, a, 1, 1, 8, 8, 4, 4, False, 1.0, 8, False)    # mask not 16-byte aligned
    d.free()


@pytest.mark.parametrize("per_head", [False, True])
def test_engine_attention_with_a_mask(eg, per_head):
    # ChannelMHA with a mask unit that multiplies element by element, through the engine mirror
    from dragon_hip.engine import IllegalArgumentException
    N, QL, VL, head, dk, dv = 2, 70, 45, 3, 16, 12
    rng = np.random.default_rng(1234 + per_head)
    KC, VC = head * dk, head * dv
    Q = rng.uniform(-1, 1, (N, QL, KC)).astype(np.float32)
    K = rng.uniform(-1, 1, (N, VL, KC)).astype(np.float32)
    V = rng.uniform(-1, 1, (N, VL, VC)).astype(np.float32)
    M = (rng.uniform(0, 1, (N, head, QL, VL) if per_head else (QL, VL)) >= 0.25).astype(np.float32) / np.float32(0.75)
    base = eg.get_param("live_blocks")
    tQ, tK, tV, tM = (eg.tensor(x, *x.shape) for x in (Q, K, V, M))
    tY = eg.attention(tQ, tK, tV, head, mask=tM)
    assert tY.dim == [N, QL, VC]
    Y = eg.valueOf(tY).reshape(N, QL, head, dv).transpose(0, 2, 1, 3)
    R = attention_masked_f64(Q.reshape(N, QL, head, dk).transpose(0, 2, 1, 3), K.reshape(N, VL, head, dk).transpose(0, 2, 1, 3),
                             V.reshape(N, VL, head, dv).transpose(0, 2, 1, 3), 1 / np.sqrt(KC),
                             np.broadcast_to(M, (N, head, QL, VL)))
    assert np.linalg.norm(Y - R) <= 1e-5 * np.linalg.norm(R)
    with pytest.raises(IllegalArgumentException):
        eg.attention(tQ, tK, tV, head, mask=eg.zeros(QL, VL + 1))          # not [QL, VL]
    with pytest.raises(IllegalArgumentException):
        eg.attention(tQ, tK, tV, head, mask=eg.zeros(N, head + 1, QL, VL))
    eg.delete(tQ, tK, tV, tM, tY)
    assert eg.get_param("live_blocks") <= base + 2          # the two rejected masks stay with the caller
