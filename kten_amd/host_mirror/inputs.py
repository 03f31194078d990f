"""Seeded synthetic inputs, specified bit by bit so any host language can regenerate them.

The reference has no seeded generator (its createRandom draws from an unseeded
java.util.Random, AbstractJVMTensorOperations.kt:41-44), so benchmark and parity inputs
come from this one:

  SplitMix64 with state = seed:  state += 0x9E3779B97F4A7C15
                                 z = state; z = (z ^ z>>30) * 0xBF58476D1CE4E5B9
                                 z = (z ^ z>>27) * 0x94D049BB133111EB;  z ^= z>>31
  u      = (z >> 40) * 2^-24                      in [0, 1), exact in fp32
  U(a,b) = a + (b - a) * u                        evaluated in fp32, one rounding per op
  N(0,1) = Box-Muller on consecutive draws (z1, z2):  u1 = ((z1 >> 40) + 1) * 2^-24,
           u2 = (z2 >> 40) * 2^-24, r = sqrt(-2 ln u1), t = 2 pi u2 in fp64; the pair
           yields r cos t then r sin t, each rounded to fp32. An odd count discards the
           last sine.
Tensors are filled in row-major order and draw from one stream in the order they are
requested.
"""
import numpy as np

_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_CHUNK = 1 << 22


class SplitMix64:
    def __init__(self, seed: int):
        self.state = np.uint64(seed & 0xFFFFFFFFFFFFFFFF)

    def next_u64(self, n: int) -> np.ndarray:
        with np.errstate(over="ignore"):
            steps = np.arange(1, n + 1, dtype=np.uint64) * _GAMMA + self.state
            self.state = steps[-1] if n else self.state
            z = steps
            z = (z ^ (z >> np.uint64(30))) * _M1
            z = (z ^ (z >> np.uint64(27))) * _M2
            z = z ^ (z >> np.uint64(31))
        return z

    def uniform(self, shape, low: float, high: float) -> np.ndarray:
        n = int(np.prod(shape, dtype=np.int64))
        out = np.empty(n, dtype=np.float32)
        lo = np.float32(low)
        span = np.float32(np.float32(high) - lo)
        for s in range(0, n, _CHUNK):
            m = min(_CHUNK, n - s)
            u = (self.next_u64(m) >> np.uint64(40)).astype(np.float32) * np.float32(2.0 ** -24)
            out[s:s + m] = lo + span * u
        return out.reshape(shape)

    def normal(self, shape) -> np.ndarray:
        n = int(np.prod(shape, dtype=np.int64))
        out = np.empty(n + (n & 1), dtype=np.float32)
        pairs = out.size // 2
        for s in range(0, pairs, _CHUNK):
            m = min(_CHUNK, pairs - s)
            z = self.next_u64(2 * m)
            u1 = ((z[0::2] >> np.uint64(40)) + np.uint64(1)).astype(np.float64) * 2.0 ** -24
            u2 = (z[1::2] >> np.uint64(40)).astype(np.float64) * 2.0 ** -24
            r = np.sqrt(-2.0 * np.log(u1))
            t = (2.0 * np.pi) * u2
            out[2 * s:2 * (s + m):2] = (r * np.cos(t)).astype(np.float32)
            out[2 * s + 1:2 * (s + m):2] = (r * np.sin(t)).astype(np.float32)
        return out[:n].reshape(shape)
