"""Philox4x32-10 and the two masks built on it.  TEST INFRASTRUCTURE ONLY.

The generator is the published one (Salmon, Moraes, Dror, Shaw: "Parallel
random numbers: as easy as 1, 2, 3", SC'11; Random123 `philox4x32_R(10, ...)`);
`tests/test_oracle_philox.py` pins this restatement with the known-answer
vectors Random123 ships (`kat_vectors`).  The reference reaches the same
generator through curand (`curand_init` / `curand_uniform4`,
megalodon/csrc/softmax.cuh:161-171) but assigns its output to elements by
CUDA thread, so its masks are not the ones below; what is restated here is the
position-based assignment this build documents in include/megalodon_hip.h.
"""
import numpy as np

_M0, _M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_W0, _W1 = 0x9E3779B9, 0xBB67AE85
_MASK = np.uint64(0xFFFFFFFF)


def philox4x32_10(counter, key):
    """counter: four broadcastable integer arrays (32-bit words), key: two ints.
    Returns an array (..., 4) of uint32."""
    c = [np.asarray(x, dtype=np.uint64) & _MASK for x in counter]
    c = list(np.broadcast_arrays(*c))
    k0, k1 = int(key[0]) & 0xFFFFFFFF, int(key[1]) & 0xFFFFFFFF
    for _ in range(10):
        p0 = _M0 * c[0]
        p1 = _M1 * c[2]
        hi0, lo0 = p0 >> np.uint64(32), p0 & _MASK
        hi1, lo1 = p1 >> np.uint64(32), p1 & _MASK
        c = [hi1 ^ c[1] ^ np.uint64(k0), lo1, hi0 ^ c[3] ^ np.uint64(k1), lo0]
        k0 = (k0 + _W0) & 0xFFFFFFFF
        k1 = (k1 + _W1) & 0xFFFFFFFF
    return np.stack(c, axis=-1).astype(np.uint32)


def uniform24(words):
    """u = (word >> 8) * 2^-24 in [0, 1), exact in float32."""
    return (words >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)


def dropkey_mask(rows, cols, p, seed, offset):
    """True where key j of row i is dropped: word j % 4 of Philox with counter
    (j // 4, i, offset lo, offset hi), key (seed lo, seed hi), u < float32(p).
    `rows`: 1-D array of global row numbers."""
    quads = np.arange((cols + 3) // 4, dtype=np.uint64)
    w = philox4x32_10((quads[None, :], np.asarray(rows, dtype=np.uint64)[:, None],
                       offset & 0xFFFFFFFF, (offset >> 32) & 0xFFFFFFFF),
                      (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    u = uniform24(w).reshape(len(rows), -1)[:, :cols]
    return u < np.float32(p)


def dropout_keep(n, p, seed, offset):
    """True where flat element e < n is kept: word e % 4 of Philox with counter
    (e // 4 lo, e // 4 hi, offset lo, offset hi), key seed, u >= float32(p)."""
    quads = np.arange((n + 3) // 4, dtype=np.uint64)
    w = philox4x32_10((quads & _MASK, quads >> np.uint64(32), offset & 0xFFFFFFFF, (offset >> 32) & 0xFFFFFFFF),
                      (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    return ~(uniform24(w).reshape(-1)[:n] < np.float32(p))
