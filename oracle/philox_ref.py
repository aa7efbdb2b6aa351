"""NumPy twin of the device dropout-mask generator.  TEST INFRASTRUCTURE ONLY.

The reference draws masks with cuRAND Philox4_32_10 seeded per thread
(``pytorch_module/blocks.cuh:24-51``, ``block_softmax.cuh:101-106``), so its bit
stream depends on the launch geometry and on the chosen layout, and cuRAND is a
closed library that is not in the reference checkout: the reference's bits are
"parity unpinned" and are not reproduced.  What is kept is the contract the
reference's own checks use (``pytorch_module/benchmark.py:304-316``): the mask
holds only 0 and 1, ``out = in * mask``, kept elements are not rescaled.

The generator restated here is the published Philox4x32-10 of Salmon et al.,
"Parallel random numbers: as easy as 1, 2, 3" (SC'11), pinned by the Random123
known-answer vectors in tests/test_oracle_philox.py.  The mapping from tensor
element to random bits is layout independent:

    e        canonical (row-major, canonical dim order) element index
    counter  (lo32(e>>3), hi32(e>>3), site, step)
    key      (lo32(seed), hi32(seed))
    r16      16-bit field (e & 7) of the 128-bit output, little-endian by word
    keep     r16 >= round(p * 65536)            (mask = 1 if keep else 0)

``site`` is 0 softmax, 1 residual-1, 2 activation, 3 residual-2; ``step`` counts
forward calls since the seed was set.
"""

import numpy as np

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_W0 = np.uint32(0x9E3779B9)
_W1 = np.uint32(0xBB67AE85)
_LO = np.uint64(0xFFFFFFFF)
_S32 = np.uint64(32)

SITE_SOFTMAX, SITE_RESID1, SITE_ACT, SITE_RESID2 = 0, 1, 2, 3


def philox4x32_10(counter, key):
    """counter: uint32 array [..., 4]; key: uint32 array [..., 2] (broadcastable).
    Returns uint32 array [..., 4]."""
    counter = np.asarray(counter, dtype=np.uint32)
    key = np.asarray(key, dtype=np.uint32)
    c0, c1, c2, c3 = (counter[..., i].copy() for i in range(4))
    k0 = np.broadcast_to(key[..., 0], c0.shape).copy()
    k1 = np.broadcast_to(key[..., 1], c0.shape).copy()
    with np.errstate(over='ignore'):
        for _ in range(10):
            p0 = _M0 * c0.astype(np.uint64)
            p1 = _M1 * c2.astype(np.uint64)
            hi0 = (p0 >> _S32).astype(np.uint32); lo0 = (p0 & _LO).astype(np.uint32)
            hi1 = (p1 >> _S32).astype(np.uint32); lo1 = (p1 & _LO).astype(np.uint32)
            c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
            k0 = (k0 + _W0).astype(np.uint32)
            k1 = (k1 + _W1).astype(np.uint32)
    return np.stack((c0, c1, c2, c3), axis=-1)


def threshold16(p):
    """Drop threshold on the 16-bit field: round(p*65536) clamped to [0, 65536].
    p is taken at float32 precision, the type the C ABI passes it in."""
    return int(min(65536, max(0, int(np.floor(float(np.float32(p)) * 65536.0 + 0.5)))))


def random16(n, seed, site, step=0, start=0):
    """The 16-bit fields for canonical element indices start .. start+n-1."""
    e = np.arange(start, start + n, dtype=np.uint64)
    g = e >> np.uint64(3)
    g0 = int(g[0]) if n else 0
    ng = (int(g[-1]) - g0 + 1) if n else 0
    gi = np.arange(g0, g0 + ng, dtype=np.uint64)
    ctr = np.empty((ng, 4), dtype=np.uint32)
    ctr[:, 0] = (gi & _LO).astype(np.uint32)
    ctr[:, 1] = (gi >> _S32).astype(np.uint32)
    ctr[:, 2] = np.uint32(site)
    ctr[:, 3] = np.uint32(step)
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint32)
    out = philox4x32_10(ctr, key)                       # [ng, 4] uint32
    # little-endian split of each word into two 16-bit fields -> [ng, 8]
    f = np.empty((ng, 8), dtype=np.uint32)
    f[:, 0::2] = out & np.uint32(0xFFFF)
    f[:, 1::2] = out >> np.uint32(16)
    f = f.reshape(-1)
    off = int(start - (g0 << 3))
    return f[off:off + n]


def dropout_mask(shape, p, seed, site, step=0, dtype=np.float32):
    """{0,1} mask of the given canonical shape (row-major canonical index)."""
    n = int(np.prod(shape))
    keep = random16(n, seed, site, step) >= np.uint32(threshold16(p))
    return keep.astype(dtype).reshape(shape)
