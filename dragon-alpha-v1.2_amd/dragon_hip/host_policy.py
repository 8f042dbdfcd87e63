"""The split-K decision of the host engine as a pure function of the compute-unit count
(reference: CudaFloat32EngineBase.java:1519-1562, 1604-1613, 1736-1779, 1855-1896), computed by the
library's C++ engine mirror.  Needs no device."""
from . import lib

MATMUL, MATMUL_T1, MATMUL_T2, MATMUL_BIASED = 0, 1, 2, 3


def gridZ(kind, N, M, K, SM):
    """GridZ for padded dims with the default knobs; 1 means no split."""
    return lib.dragon_policy_gridZ(kind, N, M, K, SM)


def smooth_maxPart(x):
    return lib.dragon_policy_smooth_maxPart(x)
