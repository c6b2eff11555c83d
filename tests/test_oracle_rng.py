"""Pins for the oracle's random streams.

Philox4x32-10: Random123 known-answer vectors (kat_vectors, philox4x32 10 rounds) and an
independent big-int Python implementation.  xorshift32: independent Python ints.
The seed/offset packing and the u32->f32 map of Mojo's step_uniform have no vector in the
reference to diff against (parity unpinned); only their internal consistency is checked.
"""
import numpy as np

M0, M1, W0, W1 = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85
MASK = 0xFFFFFFFF


def philox_py(ctr, key, rounds=10):
    c = list(ctr)
    k = list(key)
    for _ in range(rounds):
        p0, p1 = M0 * c[0], M1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & MASK, p1 & MASK, ((p0 >> 32) ^ c[3] ^ k[1]) & MASK, p0 & MASK]
        k = [(k[0] + W0) & MASK, (k[1] + W1) & MASK]
    return c


KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((MASK,) * 4, (MASK, MASK), (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
     (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


def test_philox_known_answers(orc):
    for ctr, key, want in KAT:
        assert tuple(philox_py(ctr, key)) == want
        out = np.zeros(4, np.uint32)
        orc.orc_philox4x32_10(np.array(ctr, np.uint32), np.array(key, np.uint32), out)
        assert tuple(int(v) for v in out) == want


def test_philox_uniform_matches_python(orc):
    rng = np.random.default_rng(0)
    for _ in range(200):
        seed = int(rng.integers(0, 2**63)) * 2 + int(rng.integers(0, 2))
        offset = int(rng.integers(0, 2**40))
        call = int(rng.integers(0, 20))
        out = np.zeros(4, np.float32)
        orc.orc_philox_uniform4(seed, offset, call, out)
        lo = (offset + call) & (2**64 - 1)
        raw = philox_py((lo & MASK, lo >> 32, 0, 0), (seed & MASK, seed >> 32))
        want = [np.float32(r & 0x7FFFFFFF) * np.float32(4.6566127342e-10) for r in raw]
        assert [float(v) for v in out] == [float(w) for w in want]
        assert all(0.0 <= float(v) < 1.0 for v in out)


def xorshift_py(x):
    x ^= (x << 13) & MASK
    x ^= x >> 17
    x ^= (x << 5) & MASK
    return x


def test_xorshift32_orbit(orc):
    x = 2463534242
    for _ in range(1000):
        y = xorshift_py(x)
        assert orc.orc_xorshift32(x) == y
        x = y
    assert xorshift_py(1) == 270369  # textbook first value of the 13/17/5 generator
    assert orc.orc_xorshift32(1) == 270369
