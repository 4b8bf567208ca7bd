"""tests/splitmix64.h restated for the Python tests: the same stream, the same float and integer draws, the same
checksum, so that a C++ host and a Python host that start from one seed hold identical inputs."""
import numpy as np

_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


class SplitMix64:
    def __init__(self, seed):
        self.s = np.uint64(seed)

    def next(self, n):
        """The next n outputs as a uint64 array."""
        with np.errstate(over="ignore"):
            z = self.s + _GAMMA * np.arange(1, n + 1, dtype=np.uint64)
            self.s = z[-1] if n else self.s
            z = (z ^ (z >> np.uint64(30))) * _M1
            z = (z ^ (z >> np.uint64(27))) * _M2
            return z ^ (z >> np.uint64(31))

    def uniform(self, lo, hi, n):
        """n floats: lo + (hi - lo) * u / 2^24 in single precision, each operation rounded once, in the header's order."""
        u = (self.next(n) >> np.uint64(40)).astype(np.float32)
        span = np.float32(hi) - np.float32(lo)
        return (np.float32(lo) + (span * u) / np.float32(16777216.0)).astype(np.float32)

    def integer(self, lo, hi, n):
        return (lo + (self.next(n) % np.uint64(hi - lo + 1)).astype(np.int64)).astype(np.int64)


def fnv1a64(data):
    """FNV-1a over the bytes of an array (or bytes object)."""
    b = np.frombuffer(data.tobytes() if isinstance(data, np.ndarray) else data, dtype=np.uint8)
    h = 0xCBF29CE484222325
    for chunk in np.array_split(b, max(1, b.size // 65536)):
        for v in chunk.tolist():
            h = ((h ^ v) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h
