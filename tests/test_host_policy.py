"""The host-side split-K policy of the library (C++ mirror of CudaFloat32EngineBase) against
the oracle's literal restatement and the hand-derived answers.  CPU only."""
import pytest

from oracle import oracle


def test_known_answers(dh):
    from dragon_hip import host_policy as hp
    assert hp.smooth_maxPart(256) == 128 and hp.smooth_maxPart(38) == 40 and hp.smooth_maxPart(7) == 16
    for kind in (hp.MATMUL, hp.MATMUL_T1, hp.MATMUL_T2):
        assert hp.gridZ(kind, 4096, 4096, 4096, 256) == 1          # config 2: no split
        assert hp.gridZ(kind, 1000, 780, 1532, 256) == 2           # config 5: split in two
    assert hp.gridZ(hp.MATMUL_T1, 256, 256, 131072, 256) == 128    # config 3 on 256 units
    assert hp.gridZ(hp.MATMUL_T1, 256, 256, 131072, 38) == 36      # the same on 38 units
    assert hp.gridZ(hp.MATMUL, 64, 64, 508, 256) == 1              # K below the threshold
    # matMul_biased tests blockNum against 1.2 + K/(K+1024) units where matMul uses 1.2 + 0.4*K/(K+1024):
    # 512 blocks of 2048x4096 at K = 16384 lie between 256*1.58 = 404 and 256*2.14 = 548, so only the
    # biased product splits; fGridZ = (4096 + 2048)/(2*512) = 6, capped by 256*4*0.8/512 = 1 -> raised to 2
    assert hp.gridZ(hp.MATMUL, 2048, 4096, 16384, 256) == 1
    assert hp.gridZ(hp.MATMUL_BIASED, 2048, 4096, 16384, 256) == 2
    # matMulT2's quirks (CudaFloat32EngineBase.java:1859-1867, 1894): blockNum(N, K) tested against
    # matMul's 1.2 and used as the divisor of the GridZ3 clamp.  Derivations: see
    # test_oracle_pins.test_matMulT2_policy_known_answers_that_need_its_quirks.
    assert hp.gridZ(hp.MATMUL_T2, 64, 64, 8192, 256) == 12         # 32 with blockNum(N, M) in the clamp
    assert hp.gridZ(hp.MATMUL_T1, 64, 64, 8192, 256) == 32
    assert hp.gridZ(hp.MATMUL_T2, 64, 64, 65536, 256) == 2         # 128 with blockNum(N, M) in the clamp
    assert hp.gridZ(hp.MATMUL_T1, 64, 64, 65536, 256) == 128
    assert hp.gridZ(hp.MATMUL_T2, 6784, 4, 1024, 256) == 2         # 1 with matMulT2's own 1.14


def test_policy_matches_oracle_over_a_grid(dh):
    from dragon_hip import host_policy as hp
    dims = [4, 8, 36, 64, 100, 128, 256, 260, 512, 780, 1000, 1024, 2048, 4096]
    ks = [4, 256, 508, 512, 516, 1024, 1532, 4096, 8192, 16384, 131072]
    n = 0
    for SM in (20, 38, 80, 108, 256, 304):
        for N in dims:
            for M in dims:
                for K in ks:
                    for kind in (0, 1, 2, 3):
                        assert hp.gridZ(kind, N, M, K, SM) == oracle.gridZ(kind, N, M, K, SM), \
                            (kind, N, M, K, SM)
                        n += 1
    assert n > 40000
