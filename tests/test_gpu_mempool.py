"""The device memory pool of the engine mirror against the behaviour of the reference's Memp1
(z/dragon/engine/memp/Mempool.java:150-225, Memp1.java:27-80): recycling by size, the 1.5x window,
release of buffered blocks under a tight budget, a block freed once, and no device allocation per
operation once the pool is warm."""
import numpy as np
import pytest

from helpers import oracle

pytestmark = pytest.mark.gpu

KB = 1024


@pytest.fixture()
def eg(gpu):
    from dragon_hip import engine
    e = engine.cuda_float32(0, 8, max_mem_size=4 << 20)
    yield e
    e.close()


def stats(eg):
    return tuple(eg.get_param("memp_" + k) for k in ("physical_blocks", "buffered_blocks", "used_mem_size_KB",
                                                     "total_mem_size_KB"))


def test_engine_without_a_pool_reports_none(gpu):
    from dragon_hip import engine
    e = engine.cuda_float32(0, 8)
    try:
        assert e.get_param("memp_physical_blocks") == -1
    finally:
        e.close()


def test_blocks_are_recycled_by_size(eg):
    assert stats(eg) == (0, 0, 0, 0)
    a = eg.empty(1000)                        # 4000 bytes
    addr = a.address
    assert stats(eg) == (1, 0, 3, 3)
    eg.delete(a)
    assert stats(eg) == (1, 1, 0, 3)          # buffered, still owned
    b = eg.empty(1000)
    assert b.address == addr and stats(eg) == (1, 0, 3, 3)
    eg.delete(b)
    c = eg.empty(700)                         # 2800 <= 4000 <= 1.5 * 2800: the buffered block serves it
    assert c.address == addr and stats(eg)[0] == 1
    eg.delete(c)
    d = eg.empty(600)                         # 1.5 * 2400 < 4000: too wasteful, a new block
    d_addr = d.address
    assert d_addr != addr and stats(eg)[:2] == (2, 1)
    e2 = eg.empty(1200)                       # larger than anything buffered: a new block
    assert e2.address not in (addr, d_addr) and stats(eg)[:2] == (3, 1)
    eg.delete(d, e2)
    assert stats(eg)[:3] == (3, 3, 0)
    # equal sizes: the smallest fitting block is taken
    f = eg.empty(590)                         # 2360: fits 2400 (600 floats) first
    assert f.address == d_addr
    eg.delete(f)


def test_recycled_memory_is_cleared_where_the_layout_needs_zeros(eg):
    rng = np.random.default_rng(5)
    a = eg.tensor(rng.standard_normal(30 * 8).astype(np.float32) + 7.0, 30, 8)
    addr = a.address
    eg.delete(a)
    z = eg.zeros(30, 8)
    assert z.address == addr and not eg.valueOf(z).any()
    eg.delete(z)
    # 7 columns are stored at a stride of 8: the pad of the recycled, dirty block must read as zero, or
    # the product over the padded K would pick it up
    A = rng.standard_normal((30, 7)).astype(np.float32)
    B = rng.standard_normal((7, 5)).astype(np.float32)
    tA = eg.tensor(A, 30, 7)
    assert tA.address == addr
    tB = eg.tensor(B, 7, 5)
    C = eg.valueOf(eg.matMul(tA, tB)).reshape(30, 5)
    np.testing.assert_allclose(C, oracle.matmul(0, A, B), rtol=1e-5, atol=1e-5)


def test_a_tight_budget_releases_buffered_blocks_and_then_refuses(eg):
    a = eg.empty(600 * KB // 4)               # 600 KiB of the 4 MiB budget
    b = eg.empty(3 * KB * KB // 4)            # 3 MiB
    assert stats(eg)[3] == 3672
    eg.delete(a, b)                           # both buffered
    c = eg.empty(3800 * KB // 4)              # fits neither; the budget has room only once both are released
    assert stats(eg) == (1, 0, 3800, 3800)
    with pytest.raises(RuntimeError, match="insufficient"):
        eg.empty(300 * KB // 4)               # 3800 + 300 KiB used would exceed 4 MiB
    with pytest.raises(ValueError):
        eg.empty(5 * KB * KB // 4)            # larger than the pool itself
    eg.delete(c)
    d = eg.empty(300 * KB // 4)               # now there is room: the 3800 KiB block is released for it
    assert stats(eg)[3] <= 4096
    eg.delete(d)


def test_split_k_reuses_its_partial_buffer(gpu):
    from dragon_hip import engine
    eg = engine.cuda_float32(0, 32, max_mem_size=1 << 30)
    try:
        rng = np.random.default_rng(9)
        K, N, M = 16384, 256, 256
        A = rng.standard_normal((K, N)).astype(np.float32) * 0.05
        B = rng.standard_normal((K, M)).astype(np.float32) * 0.05
        tA, tB = eg.tensor(A, K, N), eg.tensor(B, K, M)
        tC = eg.matMulT1(tA, tB)
        assert eg.get_param("last_gridZ") >= 2
        first = eg.valueOf(tC)
        warm = stats(eg)[0]
        for _ in range(3):                    # same shapes again: C and the partials come from the pool
            eg.delete(tC)
            tC = eg.matMulT1(tA, tB)
            assert np.array_equal(eg.valueOf(tC), first)
        assert stats(eg)[0] == warm           # not one more device allocation
        ref = oracle.matmul_f64(1, A, B)
        assert np.linalg.norm(first.reshape(N, M) - ref) / np.linalg.norm(ref) < 1e-5
    finally:
        eg.close()
