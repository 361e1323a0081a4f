"""Seeded synthetic tensors for the benchmark configurations.

The recipe is fixed so that every program that names a seed sees the same
data: a 64-bit Mersenne Twister (std::mt19937_64) seeded with `seed`; uniform
doubles in [0, 1) as (x >> 11) * 2^-53; normal deviates by the Box-Muller
transform on consecutive pairs (u1, u2) -> r cos t, r sin t with
r = sqrt(-2 ln(1 - u1)), t = 2 pi u2 (no library distribution: those are
implementation-defined).  Values are drawn in the order of the external
arrays: activations [B][C][field...] row-major, weights [G][Co][Ci][k...]."""
import numpy as np

_NN, _MM = 312, 156
_MATRIX_A = np.uint64(0xB5026F5AA96619E9)
_UPPER = np.uint64(0xFFFFFFFF80000000)
_LOWER = np.uint64(0x7FFFFFFF)


class MT19937_64:
    """std::mt19937_64: the 10000th output of the default seed 5489 is
    9981545732273789042 (ISO C++ [rand.predef])."""

    def __init__(self, seed=5489):
        s = np.empty(_NN, dtype=np.uint64)
        x = int(seed) & 0xFFFFFFFFFFFFFFFF
        s[0] = x
        for i in range(1, _NN):
            x = (6364136223846793005 * (x ^ (x >> 62)) + i) \
                & 0xFFFFFFFFFFFFFFFF
            s[i] = x
        self.state = s

    def _twist(self):
        s = self.state

        def mix(hi, lo):
            y = (hi & _UPPER) | (lo & _LOWER)
            return (y >> np.uint64(1)) ^ np.where(
                (y & np.uint64(1)) != 0, _MATRIX_A, np.uint64(0))

        new = np.empty_like(s)
        # new[i] = s[i + 156] ^ mix(s[i], s[i + 1]) for i < 156: old state only
        new[:_MM] = s[_MM:] ^ mix(s[:_MM], s[1:_MM + 1])
        # i in [156, 311): s[i + 156 - 312] is already new
        new[_MM:_NN - 1] = new[:_MM - 1] ^ mix(s[_MM:_NN - 1], s[_MM + 1:])
        new[_NN - 1] = new[_MM - 1] ^ mix(s[_NN - 1:], new[:1])[0]
        self.state = new

    def raw(self, n):
        """The next n 64-bit outputs."""
        blocks = -(-n // _NN)
        out = np.empty(blocks * _NN, dtype=np.uint64)
        for b in range(blocks):
            self._twist()
            y = self.state.copy()
            y ^= (y >> np.uint64(29)) & np.uint64(0x5555555555555555)
            y ^= (y << np.uint64(17)) & np.uint64(0x71D67FFFEDA60000)
            y ^= (y << np.uint64(37)) & np.uint64(0xFFF7EEE000000000)
            y ^= y >> np.uint64(43)
            out[b * _NN:(b + 1) * _NN] = y
        # (outputs of a block that are not asked for are dropped: a generator
        # is used for one array)
        return out[:n]


def uniform01(seed, n):
    return (MT19937_64(seed).raw(n) >> np.uint64(11)).astype(np.float64) \
        * 2.0 ** -53


def uniform(seed, shape, lo, hi):
    n = int(np.prod(shape))
    return (lo + (hi - lo) * uniform01(seed, n)).reshape(shape)


def normal(seed, shape, std=1.0):
    n = int(np.prod(shape))
    u = uniform01(seed, 2 * ((n + 1) // 2))
    r = np.sqrt(-2.0 * np.log1p(-u[0::2]))
    t = 2.0 * np.pi * u[1::2]
    z = np.empty(2 * r.size)
    z[0::2] = r * np.cos(t)
    z[1::2] = r * np.sin(t)
    return (std * z[:n]).reshape(shape)
