"""The drop-in boundary without a GPU: the shared library loads, exports every symbol
the public headers declare, and its host-side helpers and argument validation behave.
No compute entry point is executed here."""
import ctypes
import os
import re

import numpy as np
import pytest

from oracle import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", h) for h in ("dragon_hip_gemm.h", "dragon_hip_conv.h", "dragon_hip_runtime.h", "dragon_hip_engine.h",
                                                    "dragon_hip_testing.h")]
INVALID_VALUE = 1   # hipErrorInvalidValue


def declared_symbols():
    names = []
    for h in HEADERS:
        text = open(h).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)   # drop comments
        names += re.findall(r"\b(dragon_\w+)\s*\(", text)
    return sorted(set(names))


def test_headers_declare_something():
    names = declared_symbols()
    assert len(names) >= 60
    for must in ("dragon_Cuda_matMul_matMul", "dragon_Cuda_matMul_matMulT1SK",
                 "dragon_Cuda_matMul_SKbuf_summary", "dragon_Cuda_batchMatMul_batchMatMulT2_texture",
                 "dragon_Cuda_malloc", "dragon_Cuda_eventRecord_streams"):
        assert must in names


def test_library_exports_every_declared_symbol(dh):
    lib = ctypes.CDLL(dh._lib.LIB_PATH)
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, "declared in include/*.h but not exported: %s" % missing


def test_binding_covers_every_declared_symbol(dh):
    assert sorted(dh._lib.SIGNATURES) == declared_symbols()


def test_heuristics_match_the_oracle(dh):
    MM, BMM = dh.Cuda_matMul, dh.Cuda_batchMatMul
    for N in list(range(1, 300)) + [512, 1000, 1024, 4096, 4100]:
        for M in (1, 3, 4, 7, 64, 96, 100, 128, 255, 256, 388, 780, 4096):
            if N % 4 == 0 and M % 4 == 0:
                assert MM.blockNum(N, M) == oracle.blockNum(N, M)
                assert MM.nstream(N, M) == oracle.nstream(N, M)
            assert BMM.streamSize(N, M) == oracle.streamSize(N, M)   # N may be unpadded here
    assert MM.blockNum(4096, 4096) == 1024 and MM.nstream(1000, 780) == 10


def _streams(n):
    return (ctypes.c_int64 * max(n, 1))(*([0] * max(n, 1)))


def test_argument_validation_rejects_before_touching_the_device(dh):
    lib = dh.lib
    s = _streams(1)
    ok_ptr = 0x1000   # aligned, never dereferenced: every call below must fail validation
    f = lib.dragon_Cuda_matMul_matMul
    assert f(s, 1, 0, ok_ptr, ok_ptr, 4, 4, 4) == INVALID_VALUE          # null A
    assert f(s, 1, ok_ptr, 0, ok_ptr, 4, 4, 4) == INVALID_VALUE          # null B
    assert f(s, 1, ok_ptr, ok_ptr, 0, 4, 4, 4) == INVALID_VALUE          # null C
    assert f(s, 1, ok_ptr, ok_ptr, ok_ptr, 0, 4, 4) == INVALID_VALUE     # N <= 0
    assert f(s, 1, ok_ptr, ok_ptr, ok_ptr, 4, -4, 4) == INVALID_VALUE    # M <= 0
    assert f(s, 1, ok_ptr, ok_ptr, ok_ptr, 4, 4, 0) == INVALID_VALUE     # K <= 0
    assert f(s, 1, ok_ptr, ok_ptr, ok_ptr, 5, 4, 4) == INVALID_VALUE     # N not padded to x4
    assert f(s, 1, ok_ptr + 4, ok_ptr, ok_ptr, 4, 4, 4) == INVALID_VALUE  # misaligned
    assert f(s, 0, ok_ptr, ok_ptr, ok_ptr, 4, 4, 4) == INVALID_VALUE     # no stream
    assert f(_streams(11), 11, ok_ptr, ok_ptr, ok_ptr, 4, 4, 4) == INVALID_VALUE  # > 10 streams
    assert f(None, 1, ok_ptr, ok_ptr, ok_ptr, 4, 4, 4) == INVALID_VALUE  # null stream array
    for name in ("dragon_Cuda_matMul_matMulT1", "dragon_Cuda_matMul_matMulT2",
                 "dragon_Cuda_matMul_matMul_mma"):
        assert getattr(lib, name)(s, 1, 0, ok_ptr, ok_ptr, 4, 4, 4) == INVALID_VALUE
    sk = lib.dragon_Cuda_matMul_matMulT1SK
    assert sk(s, 1, 4, ok_ptr, ok_ptr, ok_ptr, 0, 4, 4, 64) == INVALID_VALUE   # split without Cbuf
    assert sk(s, 1, 0, ok_ptr, ok_ptr, ok_ptr, ok_ptr, 4, 4, 64) == INVALID_VALUE  # GridZ < 1
    sm = lib.dragon_Cuda_matMul_SKbuf_summary
    assert sm(0, ok_ptr, 0, 3, 64) == INVALID_VALUE
    assert sm(0, 0, ok_ptr, 3, 64) == INVALID_VALUE
    assert sm(0, ok_ptr, ok_ptr, 3, 62) == INVALID_VALUE    # sizeC not x4
    assert sm(0, ok_ptr, ok_ptr, -1, 64) == INVALID_VALUE
    b = lib.dragon_Cuda_batchMatMul_batchMatMul
    assert b(s, 1, ok_ptr, ok_ptr, ok_ptr, 0, 4, 4, 4, 4) == INVALID_VALUE      # Batch <= 0
    assert b(s, 1, ok_ptr, ok_ptr, ok_ptr, 2, 5, 6, 4, 4) == INVALID_VALUE      # M not x4
    assert b(s, 1, ok_ptr, ok_ptr, ok_ptr, 2, 5, 8, 5, 4) == INVALID_VALUE      # AK < BK
    t1 = lib.dragon_Cuda_batchMatMul_batchMatMulT1
    assert t1(s, 1, ok_ptr, ok_ptr, ok_ptr, 2, 9, 8, 4, 3) == INVALID_VALUE     # AN < CN
    t2 = lib.dragon_Cuda_batchMatMul_batchMatMulT2
    assert t2(s, 1, ok_ptr, ok_ptr, ok_ptr, 2, 5, 8, 9, 4) == INVALID_VALUE     # BM > CM
    assert t2(s, 1, ok_ptr, ok_ptr, ok_ptr, 2, 5, 8, 7, 6) == INVALID_VALUE     # K not x4
    # a row pitch beyond what 32-bit tile-local byte offsets reach (256 rows of it) is refused, not wrapped
    too_long = 1 << 21
    assert f(s, 1, ok_ptr, ok_ptr, ok_ptr, 4, 4, too_long) == INVALID_VALUE            # A's pitch = K
    assert lib.dragon_Cuda_matMul_matMulT2(s, 1, ok_ptr, ok_ptr, ok_ptr, 4, 4, too_long) == INVALID_VALUE
    assert lib.dragon_Cuda_matMul_matMulT1(s, 1, ok_ptr, ok_ptr, ok_ptr, too_long, 4, 4) == INVALID_VALUE
    assert b(s, 1, ok_ptr, ok_ptr, ok_ptr, 2, 4, 4, too_long, too_long) == INVALID_VALUE
    assert t2(s, 1, ok_ptr, ok_ptr, ok_ptr, 2, 4, 4, 4, too_long) == INVALID_VALUE


def test_paired_form_is_kept_to_spans_its_32_bit_offsets_reach(dh):
    fits = dh.lib.dragon_gemm_paired_form_fits
    NN, T1, T2 = 0, 1, 2
    assert fits(NN, 1, 4096, 4096, 4096) == 1 and fits(T1, 1, 4096, 4096, 4096) == 1
    # K-outer operands advance a whole row per k: B[K, M] of 2 GiB and more is out of reach
    assert fits(NN, 1, 64, 65536, 8188) == 1 and fits(NN, 1, 64, 65536, 8192) == 0
    assert fits(T1, 1, 65536, 64, 8192) == 0                    # A[K, N] likewise
    assert fits(T2, 1, 65536, 65536, 8192) == 1                 # both K-inner: 4 bytes per k
    assert fits(T2, 1, 4, 4, 1 << 29) == 0
    # split-K: the longest slice counts (the last one takes the remainder)
    assert fits(NN, 4, 64, 65536, 8192 * 4 - 32) == 1 and fits(NN, 4, 64, 65536, 8192 * 4) == 0
    assert fits(NN, 0, 4, 4, 4) == -1 and fits(3, 1, 4, 4, 4) == -1


def test_tile_index_divisors_divide_exactly(dh):
    """The kernels turn a tile index into (slice or batch, band, column) with multiply-and-shift pairs made
    on the host: checked against integer division at the edges of every quotient step and at random."""
    rng = np.random.default_rng(77)
    ds = list(range(1, 600)) + [2 ** k for k in range(31)] + [2 ** k + 1 for k in range(30)] + \
        [2 ** k - 1 for k in range(2, 32)] + [int(v) for v in rng.integers(1, 2 ** 31, 300)]
    mul, shift = ctypes.c_uint32(), ctypes.c_uint32()
    for d in ds:
        dh.lib.dragon_gemm_tile_divisor(d, ctypes.byref(mul), ctypes.byref(shift))
        m, s = mul.value, shift.value
        assert 2 ** 31 <= m < 2 ** 32
        ns = [0, 1, d - 1, d, d + 1, 2 ** 31 - 1, 2 ** 31 - 2] + [k * d - 1 for k in range(1, 12)] + \
            [k * d for k in range(1, 12)] + [int(v) for v in rng.integers(0, 2 ** 31, 40)]
        top = (2 ** 31 - 1) // d
        ns += [top * d, top * d - 1, top * d + d - 1]
        for n in ns:
            if 0 <= n < 2 ** 31:
                assert ((((2 * n) & 0xffffffff) * m) >> 32) >> s == n // d, (n, d)


def test_python_wrapper_raises_the_exception_type(dh):
    with pytest.raises(dh.CudaException) as e:
        dh.Cuda_matMul.matMul([0], 1, 0, 0, 0, 4, 4, 4)
    assert e.value.code == INVALID_VALUE


def test_synthetic_generator_is_the_documented_stream(dh):
    from dragon_hip import synthetic
    g = synthetic.SplitMix64(1234567)   # published splitmix64 test vector
    assert [int(v) for v in g.next(3)] == [6457827717110365317, 3203168211198807973,
                                            9817491932198370423]
    a = synthetic.stream_for(5).uniform((4, 7), -1, 1)
    b = synthetic.stream_for(5).uniform((4, 7), -1, 1)
    assert np.array_equal(a, b) and a.dtype == np.float32
    assert (a >= -1).all() and (a < 1).all()
    n = synthetic.stream_for(2).normal((200000,), 0, 1)
    assert abs(float(n.mean())) < 0.01 and abs(float(n.std()) - 1) < 0.01
    x = np.arange(15, dtype=np.float32).reshape(3, 5)
    p = synthetic.to_device_layout(x, pad_first=True)
    assert p.shape == (4, 8) and np.array_equal(p[:3, :5], x) and p[3].sum() == 0 and p[:, 5:].sum() == 0
    assert np.array_equal(synthetic.from_device_layout(p.reshape(-1), (3, 5)), x)


def test_tile_choice_on_the_documented_shapes(dh):
    # host arithmetic only.  Shape ids: 0 = 128x128, 4 = 128x64, 5 = 64x128 with 16 k per stage; 6, 8, 9 the same
    # with 32 k; 1 = 64x64, 7 = 64x64 with 32 k; 15-17 staged directly into LDS; + P: the paired-stage form,
    # taken from K = 512 on.
    NN, T1, T2 = 0, 1, 2
    P = 256
    ct = dh.choose_tile
    dh.force_tile(-1)
    # More than two 64x64 tiles per compute unit and K from 768 on: the balanced kernel with 128x128 tiles (21),
    # or with the half-size tile (19 = 128x64, 20 = 64x128; 23 = 128x64 with two workgroups per unit, where that
    # deals whole tiles) where 128x128 tiles are fewer than the units or would stand mostly empty
    for v in (NN, T1, T2):
        assert ct(v, 4096, 4096, 1, 4096) == 21 and ct(v, 8192, 4096, 1, 4096) == 21
        assert ct(v, 2816, 2816, 1, 4096) == 21 and ct(v, 2048, 2048, 1, 2048) == 21
        assert ct(v, 4096, 4096, 1, 768) == 21 and ct(v, 3000, 3000, 1, 3000) == 21
        assert ct(v, 1536, 1536, 1, 1536) == 19                   # 144 tiles of 128x128 for 256 units: 128x64
        assert ct(v, 4096, 4096, 1, 512) == P                     # a shorter K: a tile per workgroup, paired stages
        # ... except where 128x64 tiles can be dealt whole, one to three each, to two workgroups per unit (K >= 96)
        assert ct(v, 2048, 2048, 1, 512) == 23 and ct(v, 8192, 1024, 1, 512) == 23 and ct(v, 6144, 2048, 1, 256) == 23
        assert ct(v, 2048, 2048, 1, 128) == 23 and ct(v, 256, 256, 64, 128) == 23 and ct(v, 2048, 2048, 1, 80) != 23
        assert ct(v, 16384, 16384, 1, 1024) == 21                 # 16384 tiles
        assert not 18 <= ct(v, 32768 + 128, 32768, 1, 1024) < 24  # more tiles than the balanced kernel has counters for
    assert ct(T1, 256, 256, 128, 1024) == 21                      # the split-K weight gradient: 128 slices of 1024
    #                                                               are tiles like 128 batches would be
    assert ct(NN, 1024, 64, 64, 1024) == 25                       # scores x V of the attention-shaped batch: one
    #                                                               256x64 tile per unit
    assert ct(NN, 1024, 64, 64, 2048) == 23 and ct(NN, 65536, 64, 1, 1024) == 23   # otherwise 128x64, two per unit
    # A K that fits one LDS stage of 64 under a large C: the band kernel (24), from two tiles per compute unit on;
    # not for a K of 56 or less, rows of C off the 128-byte lines, or a C that leaves its tiles mostly empty
    for v in (NN, T1, T2):
        assert ct(v, 1024, 1024, 64, 64) == 24 and ct(v, 4096, 4096, 1, 60) == 24 and ct(v, 2048, 256, 64, 64) == 24
        assert ct(v, 1024, 1024, 64, 56) != 24 and ct(v, 1024, 1000, 64, 64) != 24 and ct(v, 1024, 1024, 1, 64) != 24
        assert ct(v, 130, 1024, 64, 64) != 24 and ct(v, 1024, 1024, 64, 68) != 24
    # At most two 64x64 tiles per compute unit and at least two 32-k stages per unit: the balanced kernel where its
    # estimated time is ahead (18 = one workgroup per unit; 22 = two, where only that makes the runs whole tiles)
    for v in (NN, T1, T2):
        assert ct(v, 1000, 780, 1, 1532) == 18                  # 208 tiles x 48 stages over 256 workgroups: runs of 39
        assert ct(v, 256, 256, 1, 131072) == 18                 # the tall-K weight gradient through the unsplit entry
        assert ct(v, 1024, 1024, 1, 4096) == 18 and ct(v, 512, 512, 1, 8192) == 18
        assert ct(v, 1024, 1024, 1, 1024) == 18 and ct(v, 768, 768, 1, 768) == 18 and ct(v, 512, 512, 1, 512) == 18
        assert ct(v, 2048, 1024, 1, 512) == 22                  # 512 tiles: one whole tile for each of 512 workgroups
        assert ct(v, 256, 256, 1, 256) == 17 and ct(v, 512, 512, 1, 64) == 17   # too few stages to share out
    assert ct(NN, 1000, 780, 2, 760) == 18                      # a batch of two ragged products is balanced as one
    # many tiles, a long K, runs that are not whole tiles: the half-size tile (fewer bytes staged per FLOP)
    assert ct(NN, 1000, 780, 1, 8192) == 19 and ct(NN, 768, 768, 1, 8192) == 19 and ct(NN, 1280, 1280, 1, 4096) in (19, 20)
    assert ct(NN, 640, 640, 1, 4096) == 18 and ct(NN, 1000, 780, 1, 3072) == 18 and ct(NN, 1024, 1024, 1, 4096) == 18
    # a batch of ragged products with a K of 89 ... 144: the resident-K kernel (26) where C has a rim of 1 ... 4 rows
    # or columns past a multiple of 64 and there are at least two 64x64 tiles per unit
    for v in (NN, T1, T2):
        assert ct(v, 257, 388, 36, 129) == 26 and ct(v, 257, 388, 36, 132) == 26 and ct(v, 961, 772, 4, 100) == 26
        assert ct(v, 257, 388, 36, 88) != 26 and ct(v, 257, 388, 36, 148) != 26 and ct(v, 256, 384, 36, 129) != 26
        assert ct(v, 257, 388, 8, 129) != 26                   # 192 tiles: too few
    assert ct(NN, 257, 388, 36, 64) == 1                        # a shorter K: 64x64 tiles with the rim beside them
    # a C of 4, 8, 12 or 16 columns (or rows) under at least 256 lines of the other side, one 2-D product: the skinny kernel
    for v in (NN, T1, T2):
        assert ct(v, 65536, 4, 1, 1024) == 27 and ct(v, 8, 8192, 1, 4096) == 27 and ct(v, 256, 8, 1, 4) == 27
    # 12 or 16: from 16 lines of the long side per compute unit on
    assert ct(T1, 65536, 16, 1, 1024) == 27 and ct(NN, 16, 65536, 1, 1024) == 27 and ct(T1, 12, 65536, 1, 1024) == 27
    assert ct(NN, 65536, 16, 1, 1024) == 27 and ct(T2, 16, 65536, 1, 1024) == 27 and ct(T1, 4096, 16, 1, 1024) == 27
    assert ct(NN, 4092, 16, 1, 1024) != 27 and ct(T2, 12, 2048, 1, 1024) != 27
    # 20 ... 32: from 32 lines per unit and K = 256 on; under a K of 2048 or more (cut across workgroups) 12 ... 32 from 8
    for v in (NN, T1, T2):
        assert ct(v, 8192, 32, 1, 256) == 27 and ct(v, 8192, 32, 1, 252) != 27 and ct(v, 8188, 32, 1, 1024) != 27
        assert ct(v, 2048, 32, 1, 2048) == 27 and ct(v, 16, 2048, 1, 8192) == 27 and ct(v, 2044, 12, 1, 4096) != 27
        assert ct(v, 2048, 16, 1, 2044) != 27
        assert ct(v, 256, 16, 1, 8192) == 27 and ct(v, 12, 1000, 1, 65536) == 27 and ct(v, 1024, 20, 1, 8192) != 27
    for v in (NN, T1, T2):
        assert ct(v, 65536, 36, 1, 1024) != 27 and ct(v, 65536, 20, 1, 1024) == 27 and ct(v, 4096, 20, 1, 1024) != 27 and ct(v, 65536, 4, 2, 1024) != 27 and ct(v, 252, 4, 1, 1024) != 27
    # 64x128 keeps its 16-k stages for A^T*B (both operands K-outer), takes 32-k stages otherwise
    shape = (64 * 20, 128 * 19, 1, 2048)
    if ct(NN, *shape) in (5 + P, 9 + P):
        assert ct(NN, *shape) == 9 + P and ct(T2, *shape) == 9 + P and ct(T1, *shape) == 5 + P
    assert ct(NN, 3072, 3072, 1, 512) == 7 + P                  # nine 64x64 tiles per unit: still 32-k stages
    assert ct(NN, 4096, 4096, 1, 252) == 0 and ct(NN, 4096, 4096, 1, 256) == P    # a short K keeps the plain form
    dh.force_tile(7)
    assert ct(NN, 4096, 4096, 1, 4096) == 7                     # a forced shape is reported as it is
    dh.force_tile(-1)
    assert ct(NN, 0, 4, 1, 4) == -1


def test_tile_choice_stays_inside_what_the_kernels_accept(dh):
    # host arithmetic only, over random shapes: whatever the choice is, the chosen kernel can run it -- a
    # balanced shape never has more tiles than the kernel has arrival counters, the band kernel only gets a K
    # that fits its one stage, and every id is one that exists
    rng = np.random.default_rng(20240607)
    dims = {18: (64, 64), 19: (128, 64), 20: (64, 128), 21: (128, 128), 22: (64, 64), 23: (128, 64), 25: (256, 64)}
    valid = set(range(0, 30)) | set(range(256, 266))
    dh.force_tile(-1)
    seen = set()
    for _ in range(20000):
        rows = int(rng.choice([4, 64, 256, 1000, 1024, 4096, 16384, 65536])) + int(rng.integers(0, 3)) * 4
        cols = int(rng.choice([4, 64, 128, 780, 1024, 4096, 11008, 32768])) + int(rng.integers(0, 3)) * 4
        nz = int(rng.choice([1, 1, 1, 2, 33, 64, 128, 1024]))
        k = int(rng.choice([4, 60, 64, 96, 128, 132, 256, 512, 768, 1024, 4096, 131072]))
        for v in (0, 1, 2):
            t = dh.choose_tile(v, rows, cols, nz, k, 256)
            assert t in valid, (v, rows, cols, nz, k, t)
            seen.add(t)
            if t in dims:
                bm, bn = dims[t]
                assert -(-rows // bm) * -(-cols // bn) * nz <= 65536, (v, rows, cols, nz, k, t)
            if t == 24:
                assert 56 < k <= 64 and cols % 32 == 0, (v, rows, cols, nz, k)
            if t == 26:
                assert 88 < k <= 144, (v, rows, cols, nz, k)
            if t == 27:     # the skinny kernel: one 2-D product with a C of 4 ... 16 columns (rows) and a long other side
                assert nz == 1 and ((cols in (4, 8, 12, 16) and rows >= 256) or (rows in (4, 8, 12, 16) and cols >= 256)), (v, rows, cols, nz, k)
    assert 27 in seen
    assert {21, 24} <= seen and seen & {18, 22} and seen & {19, 20, 23}      # the sample reaches every family
