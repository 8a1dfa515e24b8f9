"""CPU checks that pin the keep-mask oracle (oracle/dropout_oracle.c).

* Philox4x32-10 against the three published known-answer vectors of the Random123 distribution
  (zero, all-ones and the pi digits input; tests/golden/philox4x32_10_kat.json);
* against a second, independently written numpy implementation on random inputs;
* the mask definition: which counter / word / threshold an element uses, p = 0 keeps everything,
  per-row p, and the keep rate.
"""

import numpy as np
import pytest

from oracle import dropout as od


from tests.util import golden

KAT = [([int(x, 16) for x in v["counter"]], [int(x, 16) for x in v["key"]], [int(x, 16) for x in v["output"]])
       for v in golden("philox4x32_10_kat.json")["vectors"]]


@pytest.mark.parametrize("ctr,key,expect", KAT)
def test_philox_known_answers(ctr, key, expect):
    assert [int(x) for x in od.philox4x32_10(ctr, key)] == expect


def _philox_numpy(ctr, key):
    """Vectorised restatement written from the paper's round function, in Python integers."""
    c = [int(x) for x in ctr]
    k = [int(x) for x in key]
    m = 0xFFFFFFFF
    for _ in range(10):
        p0, p1 = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
        c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & m, (p0 >> 32) ^ c[3] ^ k[1], p0 & m]
        k = [(k[0] + 0x9E3779B9) & m, (k[1] + 0xBB67AE85) & m]
    return c


def test_philox_against_second_implementation():
    rng = np.random.default_rng(0)
    for _ in range(200):
        ctr = rng.integers(0, 2**32, 4, dtype=np.uint64)
        key = rng.integers(0, 2**32, 2, dtype=np.uint64)
        assert [int(x) for x in od.philox4x32_10(ctr, key)] == _philox_numpy(ctr, key)


def test_threshold():
    assert od.keep_threshold(0.0) == 0
    assert od.keep_threshold(0.5) == 2**15
    assert od.keep_threshold(0.25) == 2**14
    # float32(0.1) * 2^16, floored
    assert od.keep_threshold(0.1) == int(float(np.float32(0.1)) * 2**16) == 6553
    assert od.keep_threshold(float(np.nextafter(np.float32(1.0), np.float32(0.0)))) == 0xFFFF


def test_mask_definition_elementwise():
    """Element e uses counter (e // 8, 0, 0, 0), key = (seed low, seed high) and the 16-bit draw e % 8 of the
    four output words: word (e % 8) // 2, low half for even e, high half for odd e."""
    M, K, seed, p = 3, 16, 0x1234567890ABCDEF, 0.3
    mask = od.keep_mask(M, K, p, seed)
    thr = od.keep_threshold(p)
    for e in range(M * K):
        w = _philox_numpy([e // 8, 0, 0, 0], [seed & 0xFFFFFFFF, seed >> 32])
        word = w[(e % 8) // 2]
        draw = (word >> 16) if e % 2 else (word & 0xFFFF)
        assert mask.reshape(-1)[e] == (1 if draw >= thr else 0)


def test_mask_properties():
    assert od.keep_mask(8, 64, 0.0, 7).all()
    m = od.keep_mask(256, 512, 0.1, 11)
    assert abs(m.mean() - 0.9) < 0.005
    # per-row p: rows with p = 0 are all ones, the others follow their own rate; the stream does not depend on p
    row_p = np.array([0.0, 0.5] * 64, dtype=np.float32)
    mr = od.keep_mask(128, 512, row_p, 11)
    assert mr[0::2].all() and abs(mr[1::2].mean() - 0.5) < 0.01
    half = od.keep_mask(128, 512, 0.5, 11)
    assert np.array_equal(mr[1::2], half[1::2])
    # a different seed gives a different mask, the same seed the same one
    assert not np.array_equal(od.keep_mask(64, 64, 0.5, 1), od.keep_mask(64, 64, 0.5, 2))
    assert np.array_equal(od.keep_mask(64, 64, 0.5, 1), od.keep_mask(64, 64, 0.5, 1))
    # monotone in p: every element kept at p = 0.3 is kept at p = 0.1
    a, b = od.keep_mask(64, 256, 0.1, 5), od.keep_mask(64, 256, 0.3, 5)
    assert (a >= b).all()
