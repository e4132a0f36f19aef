"""The dropout pattern of the HIP kernels, restated in numpy.  TEST INFRASTRUCTURE ONLY.

The reference has no working dropout to follow (its generator, ``jvp_flash_attention/jvp_attention.py:94-122``, is
never reached: ``:2356-2357`` raises for ``dropout_p > 0``), so the pattern is this library's own: entry (z, h, i, j)
of the probabilities has the index ``((z H + h) L + i) Lk + j``; a 32-bit mix of the index and the two halves of
the 64-bit seed is compared with ``floor(p 2^32)``; the entry is kept when the mix is not below it.  Kept entries
are scaled by 1 / (1 - p), as SDPA does.  What pins this file: the library exports the pattern it uses
(``jvpfa_dropout_keep``) and the GPU tests compare it with ``keep`` bit for bit; the attention results are then
checked against ``dense`` with ``keep_scale`` from here.
"""
import numpy as np

M32 = np.uint64(0xFFFFFFFF)


def mix(idx, seed):
    """32-bit hash of the uint64 entry indices ``idx`` under a 64-bit seed (uint64 arithmetic masked to 32 bits)."""
    idx = np.asarray(idx, dtype=np.uint64)
    s0, s1 = np.uint64(seed & 0xFFFFFFFF), np.uint64((seed >> 32) & 0xFFFFFFFF)
    x = (((idx & M32) * np.uint64(0x9E3779B1)) & M32) ^ s0
    x ^= (((idx >> np.uint64(32)) * np.uint64(0x85EBCA77)) + s1) & M32
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x7FEB352D)) & M32
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x846CA68B)) & M32
    x ^= x >> np.uint64(16)
    return x


def threshold(p):
    t = float(np.float32(p)) * 4294967296.0
    return 1 if t < 1.0 else min(int(t), 4294967295)


def keep(Z, H, L, Lk, p, seed):
    """Boolean (Z, H, L, Lk): True where the probability survives."""
    if p <= 0.0:
        return np.ones((Z, H, L, Lk), dtype=bool)
    idx = np.arange(Z * H * L * Lk, dtype=np.uint64).reshape(Z, H, L, Lk)
    return mix(idx, seed) >= np.uint64(threshold(p))


def keep_scale(Z, H, L, Lk, p, seed):
    """The matrix W of ``dense``: keep / (1 - p), with 1 - p rounded as the kernels round it (fp32)."""
    if p <= 0.0:
        return None
    rinv = np.float32(1.0) / (np.float32(1.0) - np.float32(p))
    return keep(Z, H, L, Lk, p, seed) * np.float64(rinv)
