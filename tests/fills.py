"""Deterministic input fills used by the reference's own tests, restated for numpy.

These are input generators (not the algorithm under test):
  * xorshift32_unit  — tests/test_quantize.c:23-29, values ((s & 0xFFFF)/32768) - 1
  * XorShift64       — tests/test_property.c:27-42, seeds/shapes/values of the gemm property
"""
import numpy as np

M32 = 0xFFFFFFFF
M64 = 0xFFFFFFFFFFFFFFFF


def xorshift32_unit(n, seed):
    out = np.empty(n, np.float32)
    s = seed & M32
    for i in range(n):
        s ^= (s << 13) & M32
        s ^= s >> 17
        s ^= (s << 5) & M32
        out[i] = np.float32(np.float32(s & 0xFFFF) / np.float32(32768.0)) - np.float32(1.0)
    return out


class XorShift64:
    def __init__(self, seed):
        self.s = seed if seed else 0xDEADBEEF

    def next(self):
        x = self.s
        x ^= (x << 13) & M64
        x ^= x >> 7
        x ^= (x << 17) & M64
        self.s = x
        return x

    def int(self, lo, hi):
        return lo + int(self.next() % (hi - lo + 1))

    def floats(self, n, lo, hi):
        out = np.empty(n, np.float32)
        lo32, span = np.float32(lo), np.float32(hi) - np.float32(lo)
        for i in range(n):
            u = np.float32(self.next() & 0xFFFFFF) / np.float32(16777216.0)
            out[i] = lo32 + u * span
        return out


def property_case(i):
    """Case i of the reference's gemm property test: (M, N, K, A[M,K], B[K,N]) in U[-2,2)."""
    g = XorShift64((0x6E6D6D6D << 32) ^ (i + 1))
    M, N, K = g.int(1, 96), g.int(1, 96), g.int(1, 96)
    a = g.floats(M * K, -2.0, 2.0).reshape(M, K)
    b = g.floats(K * N, -2.0, 2.0).reshape(K, N)
    return M, N, K, a, b
