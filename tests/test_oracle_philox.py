"""Pins oracle/philox_ref.py: Random123 known-answer vectors for philox4x32_10
(kat_vectors of the Random123 distribution, Salmon et al. SC'11) and the
element -> bits mapping."""
import numpy as np

from oracle import philox_ref as ph

KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


def test_philox_known_answers():
    for ctr, key, want in KAT:
        got = ph.philox4x32_10(np.array(ctr, dtype=np.uint32), np.array(key, dtype=np.uint32))
        assert tuple(int(v) for v in got) == want


def test_philox_vectorised_matches_scalar():
    ctr = np.array([k[0] for k in KAT], dtype=np.uint32)
    key = np.array([k[1] for k in KAT], dtype=np.uint32)
    got = ph.philox4x32_10(ctr, key)
    for i, (_, _, want) in enumerate(KAT):
        assert tuple(int(v) for v in got[i]) == want


def _philox_scalar(ctr, key):
    """Independent pure-Python Philox4x32-10 (textbook form)."""
    c = list(ctr); k = list(key)
    for _ in range(10):
        p0 = 0xD2511F53 * c[0]; p1 = 0xCD9E8D57 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xffffffff, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xffffffff]
        k = [(k[0] + 0x9E3779B9) & 0xffffffff, (k[1] + 0xBB67AE85) & 0xffffffff]
    return c


def test_random16_field_mapping():
    seed, site, step = 0x123456789abcdef0, 2, 5
    r = ph.random16(40, seed, site, step, start=3)
    for i, e in enumerate(range(3, 43)):
        g = e >> 3
        out = _philox_scalar([g & 0xffffffff, g >> 32, site, step],
                             [seed & 0xffffffff, seed >> 32])
        lane = e & 7
        word = out[lane >> 1]
        want = (word >> 16) if (lane & 1) else (word & 0xffff)
        assert int(r[i]) == want


def test_mask_statistics_and_extremes():
    m = ph.dropout_mask((64, 1024), 0.1, seed=7, site=0)
    assert set(np.unique(m)) == {0.0, 1.0}
    assert abs(1.0 - m.mean() - 0.1) < 5e-3
    assert ph.dropout_mask((1000,), 0.0, 1, 1).min() == 1.0
    assert ph.dropout_mask((1000,), 1.0, 1, 1).max() == 0.0
    # different site / step / seed give different masks; same args reproduce
    a = ph.dropout_mask((4096,), 0.5, 3, 0, 0)
    assert (a == ph.dropout_mask((4096,), 0.5, 3, 0, 0)).all()
    for other in (ph.dropout_mask((4096,), 0.5, 3, 1, 0), ph.dropout_mask((4096,), 0.5, 3, 0, 1),
                  ph.dropout_mask((4096,), 0.5, 4, 0, 0)):
        assert 0.4 < (a != other).mean() < 0.6


def test_threshold():
    assert ph.threshold16(0.0) == 0 and ph.threshold16(1.0) == 65536
    assert ph.threshold16(0.1) == 6554 and ph.threshold16(0.5) == 32768
