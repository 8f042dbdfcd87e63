"""Seeded synthetic inputs and Dragon tensor layout helpers for benchmarks and tests.

Generator: one splitmix64 stream per workload, seed = 0xD7A60000 + workload number,
A drawn before B, values in logical row-major order.  Uniform(a,b) uses the top 24 bits
of each 64-bit output; Normal(mu, sigma) is Box-Muller in float64 on pairs of consecutive
outputs (both branches used), rounded to float32.  The stream is counter-based, so it is computed in bulk.

Layout (reference: source/alpha-Dragon-v1.2/src/z/dragon/engine/Tensor.java:206-239,
EngineCore.java:708-810): row-major float32, the last dimension padded with zeros to a
multiple of 4 (the memory stride); allocations also round the first dimension up to a
multiple of 4.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
SEED_BASE = 0xD7A60000


class SplitMix64:
    def __init__(self, seed):
        self.state = np.uint64(seed)

    def next(self, n):
        """n consecutive 64-bit outputs."""
        with np.errstate(over="ignore"):
            idx = np.arange(1, n + 1, dtype=np.uint64)
            z = self.state + idx * _GOLDEN
            self.state = self.state + np.uint64(n) * _GOLDEN
            z = (z ^ (z >> np.uint64(30))) * _M1
            z = (z ^ (z >> np.uint64(27))) * _M2
            z = z ^ (z >> np.uint64(31))
        return z

    def uniform(self, shape, lo, hi):
        n = int(np.prod(shape))
        u = (self.next(n) >> np.uint64(40)).astype(np.float64) * (1.0 / (1 << 24))
        return (lo + (hi - lo) * u).astype(np.float32).reshape(shape)

    def normal(self, shape, mu, sigma):
        """Box-Muller on consecutive output pairs (z0, z1): u1 = ((z0 >> 11) + 1) / 2^53 in
        (0, 1], u2 = (z1 >> 11) / 2^53; the pair yields r*cos(2 pi u2) then r*sin(2 pi u2)
        with r = sqrt(-2 ln u1).  An odd count drops the last sine."""
        n = int(np.prod(shape))
        pairs = (n + 1) // 2
        z = self.next(2 * pairs)
        u1 = ((z[0::2] >> np.uint64(11)).astype(np.float64) + 1.0) * (1.0 / (1 << 53))
        u2 = (z[1::2] >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))
        del z
        r = np.sqrt(-2.0 * np.log(u1))
        ang = 2.0 * np.pi * u2
        g = np.empty(2 * pairs, dtype=np.float32)
        g[0::2] = mu + sigma * (r * np.cos(ang))
        g[1::2] = mu + sigma * (r * np.sin(ang))
        return g[:n].reshape(shape)


def stream_for(workload):
    return SplitMix64(SEED_BASE + int(workload))


def pad4(n):
    return (int(n) + 3) >> 2 << 2


def to_device_layout(x, pad_first=False):
    """Logical array -> the flat padded buffer the engine sees: last dim zero-padded to
    a multiple of 4; with pad_first the leading dim is rounded up too (zero rows)."""
    x = np.asarray(x, dtype=np.float32)
    shape = list(x.shape)
    shape[-1] = pad4(shape[-1])
    if pad_first:
        shape[0] = pad4(shape[0])
    out = np.zeros(shape, dtype=np.float32)
    out[tuple(slice(0, s) for s in x.shape)] = x
    return out


def from_device_layout(buf, shape):
    """Flat padded buffer -> logical array of `shape` (drops the padding)."""
    shape = tuple(int(s) for s in shape)
    padded = list(shape)
    padded[-1] = pad4(shape[-1])
    n = int(np.prod(padded))
    v = np.asarray(buf, dtype=np.float32).reshape(-1)[:n].reshape(padded)
    return v[..., :shape[-1]]
