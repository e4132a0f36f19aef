"""The dropout pattern of the HIP kernels, restated in numpy.  TEST INFRASTRUCTURE ONLY.

The reference has no working dropout to follow (its generator, ``jvp_flash_attention/jvp_attention.py:94-122``, is
never reached: ``:2356-2357`` raises for ``dropout_p > 0``), so the pattern is this library's own.  Query rows are
taken in blocks of 32: the block index ``(z H + h) ceil(L / 32) + i // 32`` and the two halves of the 64-bit seed go
through a 64 -> 32 bit mix; inside a block the word moves by one constant per row and another per key, and two
multiply-xorshift rounds finish it; the result is compared with ``floor(p 2^32)`` and the entry is kept when it is not
below.  Kept entries are scaled by 1 / (1 - p), as SDPA does.  What pins this file: the library exports the pattern it
uses (``jvpfa_dropout_keep``) and the GPU tests compare it with ``keep`` bit for bit; the attention results are then
checked against ``dense`` with ``keep_scale`` from here.
"""
import numpy as np

M32 = np.uint64(0xFFFFFFFF)
C_KEY, C_ROW = np.uint64(0x9E3779B1), np.uint64(0x85EBCA77)


def mix(idx, seed):
    """32-bit hash of the uint64 block indices ``idx`` under a 64-bit seed (uint64 arithmetic masked to 32 bits)."""
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


def finish(x):
    """The two rounds that turn an entry's word into its hash (a bijection of the 32-bit words)."""
    x = np.asarray(x, dtype=np.uint64) & M32
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x7FEB352D)) & M32
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x846CA68B)) & M32
    return x


def entry_hash(zh, i, j, L, seed):
    """Hash of entry (head ``zh`` = z H + h, query ``i``, key ``j``); the arguments broadcast against each other."""
    zh, i, j = (np.asarray(a, dtype=np.uint64) for a in (zh, i, j))
    block = zh * np.uint64((L + 31) // 32) + (i >> np.uint64(5))
    return finish(mix(block, seed) + (i & np.uint64(31)) * C_ROW + ((j * C_KEY) & M32))


def threshold(p):
    t = float(np.float32(p)) * 4294967296.0
    return 1 if t < 1.0 else min(int(t), 4294967295)


def keep(Z, H, L, Lk, p, seed):
    """Boolean (Z, H, L, Lk): True where the probability survives."""
    if p <= 0.0:
        return np.ones((Z, H, L, Lk), dtype=bool)
    zh = np.arange(Z * H, dtype=np.uint64)[:, None, None]
    i, j = np.arange(L, dtype=np.uint64)[None, :, None], np.arange(Lk, dtype=np.uint64)[None, None, :]
    return (entry_hash(zh, i, j, L, seed) >= np.uint64(threshold(p))).reshape(Z, H, L, Lk)


def keep_scale(Z, H, L, Lk, p, seed):
    """The matrix W of ``dense``: keep / (1 - p), with 1 - p rounded as the kernels round it (fp32)."""
    if p <= 0.0:
        return None
    rinv = np.float32(1.0) / (np.float32(1.0) - np.float32(p))
    return keep(Z, H, L, Lk, p, seed) * np.float64(rinv)
