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

import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_W0 = np.uint64(0x9E3779B9)
_W1 = np.uint64(0xBB67AE85)
_LO = np.uint64(0xFFFFFFFF)
_S32 = np.uint64(32)

SITE_SOFTMAX, SITE_RESID1, SITE_ACT, SITE_RESID2 = 0, 1, 2, 3


def philox4x32_10(counter, key):
    """counter: uint32 array [..., 4]; key: uint32 array [..., 2] (broadcastable).
    Returns uint32 array [..., 4].  The four words are carried in uint64 lanes so
    that the 32x32 -> 64 bit products need no conversions."""
    counter = np.asarray(counter, dtype=np.uint32)
    key = np.asarray(key, dtype=np.uint32)
    c0, c1, c2, c3 = (counter[..., i].astype(np.uint64) for i in range(4))
    k0 = np.broadcast_to(key[..., 0], c0.shape).astype(np.uint64)
    k1 = np.broadcast_to(key[..., 1], c0.shape).astype(np.uint64)
    for _ in range(10):
        p0 = _M0 * c0
        p1 = _M1 * c2
        c0, c1, c2, c3 = (p1 >> _S32) ^ c1 ^ k0, p1 & _LO, (p0 >> _S32) ^ c3 ^ k1, p0 & _LO
        k0 = (k0 + _W0) & _LO
        k1 = (k1 + _W1) & _LO
    return np.stack((c0, c1, c2, c3), axis=-1).astype(np.uint32)


def threshold16(p):
    """Drop threshold on the 16-bit field: round(p*65536) clamped to [0, 65536].
    p is taken at float32 precision, the type the C ABI passes it in."""
    return int(min(65536, max(0, int(np.floor(float(np.float32(p)) * 65536.0 + 0.5)))))


_CHUNK = 1 << 18      # counter groups per call of philox4x32_10: the working set stays in cache


def _fields(g0, ng, seed, site, step):
    """The 8 * ng 16-bit fields of counter groups g0 .. g0+ng-1 (uint16)."""
    gi = np.arange(g0, g0 + ng, dtype=np.uint64)
    ctr = np.empty((ng, 4), dtype=np.uint32)
    ctr[:, 0] = (gi & _LO).astype(np.uint32)
    ctr[:, 1] = (gi >> _S32).astype(np.uint32)
    ctr[:, 2] = np.uint32(site)
    ctr[:, 3] = np.uint32(step)
    key = np.array([seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF], dtype=np.uint32)
    out = philox4x32_10(ctr, key)                       # [ng, 4] uint32
    # little-endian split of each word into two 16-bit fields -> [ng, 8]
    f = np.empty((ng, 8), dtype=np.uint16)
    f[:, 0::2] = out & np.uint32(0xFFFF)
    f[:, 1::2] = out >> np.uint32(16)
    return f.reshape(-1)


def _chunked(n, start, seed, site, step, out, convert):
    """Fills out[0:n] with convert(fields) of elements start .. start+n-1, chunk by
    chunk on a few threads (NumPy releases the interpreter lock in these loops)."""
    if n == 0:
        return
    g_first, g_last = start >> 3, (start + n - 1) >> 3
    jobs = [(g, min(_CHUNK, g_last + 1 - g)) for g in range(g_first, g_last + 1, _CHUNK)]

    def run(job):
        g0, ng = job
        f = _fields(g0, ng, seed, site, step)
        lo = max(start, g0 << 3); hi = min(start + n, (g0 + ng) << 3)
        out[lo - start:hi - start] = convert(f[lo - (g0 << 3):hi - (g0 << 3)])

    workers = min(len(jobs), os.cpu_count() or 1, 16)
    if workers <= 1:
        for job in jobs:
            run(job)
    else:
        with ThreadPoolExecutor(max_workers=workers) as ex:
            list(ex.map(run, jobs))


def random16(n, seed, site, step=0, start=0):
    """The 16-bit fields for canonical element indices start .. start+n-1."""
    out = np.empty(n, dtype=np.uint32)
    _chunked(n, start, seed, site, step, out, lambda f: f)
    return out


def dropout_mask(shape, p, seed, site, step=0, dtype=np.float32):
    """{0,1} mask of the given canonical shape (row-major canonical index)."""
    n = int(np.prod(shape))
    thr = threshold16(p)
    out = np.empty(n, dtype=dtype)
    _chunked(n, 0, seed, site, step, out, lambda f: f.astype(np.uint32) >= thr)
    return out.reshape(shape)
