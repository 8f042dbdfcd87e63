"""Callers the reference does not have but a serving loop does: several host threads driving the
C ABI at once on their own streams, and launches recorded into a HIP graph and replayed.
The entry points keep no per-call host state and allocate nothing, so both must give the bits of
a plain call."""
import threading

import numpy as np
import pytest

from helpers import pad2

pytestmark = pytest.mark.gpu


def test_host_threads_on_their_own_streams(dh, gpu):
    Cuda, MM, BMM = dh.Cuda, dh.Cuda_matMul, dh.Cuda_batchMatMul
    rng = np.random.default_rng(0)
    shapes = [(130, 203, 77), (257, 64, 516), (64, 1000, 33), (512, 512, 512), (1000, 780, 1532), (33, 45, 29)]
    cases = []
    for (N, M, K) in shapes:
        A = pad2(rng.integers(-3, 4, (N, K)).astype(np.float32))        # integers: every order exact
        B = pad2(rng.integers(-3, 4, (K, M)).astype(np.float32))
        cases.append((A, B, (A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32)))
    errors = []

    def worker(idx):
        try:
            A, B, R = cases[idx]
            stream = Cuda.newStream_NonBlocking()
            dA, dB = dh.DeviceArray(A), dh.DeviceArray(B)
            dC = dh.DeviceArray(size=R.size)
            N4, K4, M4 = A.shape[0], A.shape[1], B.shape[1]
            for it in range(20):
                gz = 1 + (it % 3)
                if gz == 1:
                    MM.matMul([stream], 1, dA.address, dB.address, dC.address, N4, M4, K4)
                else:
                    dCb = dh.DeviceArray(size=R.size * (gz - 1))
                    MM.matMulSK([stream], 1, gz, dA.address, dB.address, dC.address, dCb.address, N4, M4, K4)
                    MM.SKbuf_summary(stream, dCb.address, dC.address, gz - 1, R.size)
                Cuda.streamSynchronize(stream)
                if gz > 1:
                    dCb.free()
                out = np.empty(R.size, np.float32)
                Cuda.get1D(stream, dC.address, out, R.size)
                if not np.array_equal(out.reshape(R.shape), R):
                    errors.append((idx, it, "mismatch"))
            for d in (dA, dB, dC):
                d.free()
            Cuda.deleteStream(stream)
        except Exception as e:   # noqa: BLE001 - reported below
            errors.append((idx, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(cases))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_launches_replay_from_a_hip_graph(gpu):
    # Graph capture goes through torch (its stream and graph objects), and torch has to be imported
    # before the library: both bring a HIP runtime of the same name and the process keeps the first.
    # So the check runs in a process of its own (tests/graph_replay_check.py).
    import os
    import subprocess
    import sys
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "graph_replay_check.py")
    r = subprocess.run([sys.executable, script], capture_output=True, text=True, timeout=600)
    if r.returncode == 77:
        pytest.skip(r.stdout.strip() or "torch with a GPU is not available")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "graph replay ok" in r.stdout
