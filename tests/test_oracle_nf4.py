"""Pins the NF4 dequantisation oracle (C restatement, oracle/nf4_oracle.c).

* the 16 code values are the reference's constants (dequantize_nf4.py:16-33), bit for bit;
* brute force: every 4-bit code x every 8-bit absmax code against exact rational arithmetic with a
  hand-written round-to-nearest-even (one rounding per fp32 op: the fma, then the product, then bf16);
* a case where fused multiply-add and multiply-then-add differ, so a restatement that rounds twice fails;
* nibble order, block indexing across a second-level boundary, the non-nested special case;
* round trip: |dequant(quant(w)) - w| bounded by half the widest code gap (0.3038 between -1 and -0.6962) times absmax.
"""

import numpy as np

from oracle import nf4
from tests.util import golden


def test_code_table_bits():
    expect = [float(v) for v in golden("nf4_code_table.json")["values"]]
    assert nf4.NF4_CODE.dtype == np.float32
    assert np.array_equal(nf4.NF4_CODE, np.asarray(expect, dtype=np.float32))
    lib_table = np.ctypeslib.as_array(nf4._lib().nf4_code_table(), shape=(16,))
    assert np.array_equal(lib_table.view(np.uint32), nf4.NF4_CODE.view(np.uint32))
    assert nf4.NF4_CODE[0] == -1 and nf4.NF4_CODE[7] == 0 and nf4.NF4_CODE[15] == 1
    assert (np.diff(nf4.NF4_CODE) > 0).all()


def test_bruteforce_all_codes_exact_rational():
    rng = np.random.default_rng(0)
    code2 = nf4.dynamic_code_table()
    # 256 blocks of 64 elements: block b uses absmax code b; every 4-bit code appears in every block
    n = 256 * 64
    idx = np.tile(np.arange(16, dtype=np.uint8), n // 16)
    rng.shuffle(idx.reshape(256, 64), axis=1)
    packed = ((idx[0::2] << 4) | idx[1::2]).astype(np.uint8)
    st = nf4.NF4State(packed, (n,), 64, np.arange(256, dtype=np.uint8), code2,
                      np.asarray([0.0371], dtype=np.float32), np.asarray([0.0213], dtype=np.float32))
    assert np.array_equal(nf4.dequantize(st), nf4.dequantize_exact(st))


def test_fma_is_single_rounding():
    # choose code*absmax2 + offset so that rounding the product first changes the fp32 result
    rng = np.random.default_rng(1)
    found = 0
    for _ in range(20000):
        c, a2, off = (np.float32(v) for v in rng.uniform(0.01, 1.0, 3))
        two_step = np.float32(np.float32(c * a2) + off)
        exact = nf4._round_fraction_to_f32(nf4.Fraction(float(c)) * nf4.Fraction(float(a2)) + nf4.Fraction(float(off)))
        if two_step != exact:
            code2 = np.zeros(256, dtype=np.float32)
            code2[5] = c
            st = nf4.NF4State(np.full(32, 0xFF, dtype=np.uint8), (64,), 64, np.asarray([5], dtype=np.uint8), code2,
                              np.asarray([a2], dtype=np.float32), np.asarray([off], dtype=np.float32))
            _, f32 = nf4.dequantize(st, want_f32=True)
            assert f32[0] == exact and f32[0] != two_step     # code 15 = 1.0 -> the value is absmax itself
            found += 1
            if found == 5:
                break
    assert found == 5


def test_nibble_order_and_block_indexing():
    code2 = np.linspace(0.0, 1.0, 256, dtype=np.float32)
    n = 64 * 512            # 512 first-level blocks -> 2 second-level blocks
    packed = np.zeros(n // 2, dtype=np.uint8)
    packed[0] = 0xF0        # element 0 <- high nibble (code 15 = +1), element 1 <- low nibble (code 0 = -1)
    packed[32] = 0x0F       # first byte of block 1: element 64 = -1, element 65 = +1
    absq = np.full(512, 255, dtype=np.uint8)
    absq[1] = 128
    absmax2 = np.asarray([2.0, 8.0], dtype=np.float32)
    packed[(256 * 64) // 2] = 0xFF    # first byte of the second second-level block
    st = nf4.NF4State(packed, (n,), 64, absq, code2, absmax2, np.asarray([0.5], dtype=np.float32))
    _, f = nf4.dequantize(st, want_f32=True)
    assert f[0] == 2.5 and f[1] == -2.5                        # 1.0*2.0 + 0.5
    a1 = np.float32(code2[128]) * np.float32(2.0) + np.float32(0.5)
    assert f[64] == -a1 and f[65] == a1
    assert f[256 * 64] == 8.5 and f[256 * 64 + 1] == 8.5       # uses absmax2[1]
    assert f[2] == np.float32(nf4.NF4_CODE[0]) * np.float32(2.5)   # untouched bytes are code 0 = -1


def test_non_nested_reduces_to_lut_times_absmax():
    rng = np.random.default_rng(2)
    packed = rng.integers(0, 256, 64, dtype=np.uint8)
    absmax = rng.uniform(0.01, 3.0, 4).astype(np.float32)
    st = nf4.NF4State(packed, (128,), 32, absmax, None, None, None)
    bits, f = nf4.dequantize(st, want_f32=True)
    idx = np.stack([packed >> 4, packed & 15], axis=1).reshape(-1)
    expect = nf4.NF4_CODE[idx] * np.repeat(absmax, 32)
    assert np.array_equal(f, expect.astype(np.float32))
    assert np.array_equal(bits, nf4.dequantize_exact(st))


def test_bf16_rounding_is_nearest_even():
    # a value exactly half-way between two bf16 numbers must round to the even one
    code2 = np.zeros(256, dtype=np.float32)
    code2[1] = 1.0
    for absmax, expect_bits in ((np.float32(1.00390625), 0x3F80), (np.float32(1.01171875), 0x3F82)):
        st = nf4.NF4State(np.full(32, 0xFF, dtype=np.uint8), (64,), 64, np.asarray([1], dtype=np.uint8), code2,
                          np.asarray([absmax], dtype=np.float32), np.asarray([0.0], dtype=np.float32))
        assert int(nf4.dequantize(st)[0]) == expect_bits


def test_round_trip_error_bound():
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((256, 1024)) * 0.02).astype(np.float32)
    for nested in (True, False):
        st = nf4.quantize_nf4(w, nested=nested)
        _, f = nf4.dequantize(st, want_f32=True)
        absmax = np.abs(w.reshape(-1, 64)).max(axis=1)
        err = np.abs(f.reshape(-1, 64) - w.reshape(-1, 64)).max(axis=1)
        slack = 0.03 if nested else 1e-6
        assert (err <= (0.1520 + slack) * absmax + 1e-7).all()  # widest code gap: -1.0 .. -0.6962, half of it
    assert st.packed.dtype == np.uint8 and st.packed.size == w.size // 2
