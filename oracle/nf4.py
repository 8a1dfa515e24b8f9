"""NF4 oracle, Python side (test infrastructure).

``dequantize`` calls the C restatement in ``nf4_oracle.c`` (single-rounding ``fmaf``).
``dequantize_exact`` re-derives the same values with exact rational arithmetic and a
hand-written round-to-nearest-even, for pinning the C code on small inputs.

``quantize_nf4`` and ``dynamic_code_table`` generate test inputs.  The reference obtains
them from ``bitsandbytes.functional.quantize_4bit`` (call sites
/root/reference/lorafusion/ops/triton_ops/experimental/fused_quantized_nf4_lora_xw_sb.py:38-43),
a dependency that is neither vendored nor version-pinned there: **parity unpinned** for
these two.  The dequantiser does not depend on them -- codes, absmax and the 256-entry
table are its *inputs*.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from dataclasses import dataclass
from fractions import Fraction

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

# lorafusion/ops/triton_ops/dequantize_nf4.py:16-33
NF4_CODE = np.array(
    [-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
     -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
     0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
     0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0],
    dtype=np.float32,
)


def build(force: bool = False) -> str:
    path = os.path.join(_HERE, "libnf4_oracle.so")
    if force or not os.path.exists(path):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return path


def _lib():
    global _LIB
    if _LIB is None:
        lib = ctypes.CDLL(build())
        lib.nf4_dequant_ref.restype = None
        lib.nf4_dequant_ref.argtypes = [ctypes.c_void_p] * 8 + [ctypes.c_int64, ctypes.c_int, ctypes.c_int]
        lib.routing_table_ref.restype = ctypes.c_int64
        lib.routing_table_ref.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                          ctypes.c_void_p, ctypes.c_int64]
        lib.nf4_code_table.restype = ctypes.POINTER(ctypes.c_float)
        _LIB = lib
    return _LIB


@dataclass
class NF4State:
    """The tensors a bitsandbytes ``QuantState`` carries for an NF4 weight
    (dequantize_nf4.py:271-315 reads .shape .blocksize .absmax .offset .state2.{code,absmax,blocksize})."""

    packed: np.ndarray        # uint8 [n/2]
    shape: tuple
    blocksize: int
    absmax: np.ndarray        # uint8 [n/blocksize] when nested, else float32
    code2: np.ndarray | None  # float32 [256]
    absmax2: np.ndarray | None  # float32 [n/blocksize/blocksize2]
    offset: np.ndarray | None   # float32 [1]
    blocksize2: int = 256

    @property
    def nested(self) -> bool:
        return self.absmax2 is not None


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def dequantize(st: NF4State, want_f32: bool = False):
    """C-oracle dequant.  Returns bf16 bit patterns (uint16 [n]) and optionally the fp32 products."""
    n = int(np.prod(st.shape))
    out16 = np.empty(n, dtype=np.uint16)
    out32 = np.empty(n, dtype=np.float32) if want_f32 else None
    packed = np.ascontiguousarray(st.packed, dtype=np.uint8)
    if st.nested:
        absq = np.ascontiguousarray(st.absmax, dtype=np.uint8)
        _lib().nf4_dequant_ref(_ptr(packed), _ptr(absq), None, _ptr(st.code2), _ptr(st.absmax2), _ptr(st.offset),
                               _ptr(out32), _ptr(out16), n, st.blocksize, st.blocksize2)
    else:
        am = np.ascontiguousarray(st.absmax, dtype=np.float32)
        _lib().nf4_dequant_ref(_ptr(packed), None, _ptr(am), None, None, None, _ptr(out32), _ptr(out16),
                               n, st.blocksize, 0)
    return (out16, out32) if want_f32 else out16


def routing_table_c(seq_len_list, rank_list, block_size_m):
    seq = np.asarray(seq_len_list, dtype=np.int32)
    rk = np.asarray(rank_list, dtype=np.int32)
    nb = int(sum(((int(s) - 1) // block_size_m + 1) for s in seq_len_list))
    out = np.zeros((nb, 3), dtype=np.int32)
    got = _lib().routing_table_ref(_ptr(seq), _ptr(rk), len(seq), block_size_m, _ptr(out), nb)
    if got != nb:
        raise ValueError(f"Expected {nb} blocks, but filled {got}")
    return out


# ------------------------------------------------------------------ exact cross-check


def _round_fraction_to_f32(x: Fraction) -> np.float32:
    """Round an exact rational to the nearest fp32 (ties to even); normal + subnormal range."""
    if x == 0:
        return np.float32(0.0)
    sign = -1 if x < 0 else 1
    x = abs(x)
    e = 0
    # find e with 2^e <= x < 2^(e+1)
    while Fraction(2) ** (e + 1) <= x:
        e += 1
    while Fraction(2) ** e > x:
        e -= 1
    e = max(e, -126)
    ulp = Fraction(2) ** (e - 23)
    qf = x / ulp
    qi = qf.numerator // qf.denominator
    rem = qf - qi
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (qi & 1)):
        qi += 1
    return np.float32(sign * float(Fraction(qi) * ulp))  # exact: qi*ulp is representable


def _f32_to_bf16_bits_exact(v: np.float32) -> int:
    u = int(np.asarray(v, dtype=np.float32).view(np.uint32))
    lower = u & 0xFFFF
    upper = u >> 16
    if lower > 0x8000 or (lower == 0x8000 and (upper & 1)):
        upper += 1
    return upper & 0xFFFF


def dequantize_exact(st: NF4State) -> np.ndarray:
    """Slow exact restatement (rationals; one rounding per fp32 op) -> bf16 bits.  Small inputs only."""
    n = int(np.prod(st.shape))
    out = np.empty(n, dtype=np.uint16)
    for e in range(n):
        byte = int(st.packed[e // 2])
        idx = (byte >> 4) if (e % 2 == 0) else (byte & 15)
        blk = e // st.blocksize
        if st.nested:
            prod = Fraction(float(st.code2[int(st.absmax[blk])])) * Fraction(float(st.absmax2[blk // st.blocksize2]))
            absmax = _round_fraction_to_f32(prod + Fraction(float(st.offset[0])))
        else:
            absmax = np.float32(st.absmax[blk])
        val = _round_fraction_to_f32(Fraction(float(NF4_CODE[idx])) * Fraction(float(absmax)))
        bits = _f32_to_bf16_bits_exact(val)
        if val == 0 and (np.signbit(NF4_CODE[idx]) != np.signbit(absmax)):
            bits |= 0x8000  # IEEE sign of a zero product: code 7 (+0.0) times a negative absmax is -0.0
        out[e] = bits
    return out


# ------------------------------------------------------------------ input generators (parity unpinned)


def dynamic_code_table(signed: bool = True, max_exponent_bits: int = 7, total_bits: int = 8) -> np.ndarray:
    """A 256-entry signed dynamic-exponent table in the style bitsandbytes uses for the
    second-level absmax codes.  Generated from its published description, not checked
    against the library: parity unpinned.  Sorted ascending, contains 0 and +/-1."""
    data = []
    non_sign_bits = total_bits - 1
    additional_items = 2 ** (non_sign_bits - max_exponent_bits) - 1
    for i in range(max_exponent_bits):
        fraction_items = 2 ** (i + non_sign_bits - max_exponent_bits) + 1
        boundaries = np.linspace(0.1, 1, fraction_items)
        means = (boundaries[:-1] + boundaries[1:]) / 2.0
        data += (10.0 ** (-(max_exponent_bits - 1) + i) * means).tolist()
        if signed:
            data += (-(10.0 ** (-(max_exponent_bits - 1) + i)) * means).tolist()
    if additional_items > 0:
        boundaries = np.linspace(0.1, 1, additional_items + 1)
        means = (boundaries[:-1] + boundaries[1:]) / 2.0
        data += (10.0 ** (-(max_exponent_bits - 1) + max_exponent_bits - 1) * means).tolist()
        if signed:
            data += (-(10.0 ** (-(max_exponent_bits - 1) + max_exponent_bits - 1)) * means).tolist()
    data += [0.0, 1.0]
    data += [0.0] * (2 ** total_bits - len(data))
    return np.sort(np.asarray(data, dtype=np.float32))


def _nearest_code(x: np.ndarray, table: np.ndarray) -> np.ndarray:
    """Index of the nearest table entry (table sorted ascending); ties go to the lower index."""
    mids = (table[:-1].astype(np.float64) + table[1:].astype(np.float64)) / 2.0
    return np.searchsorted(mids, x.astype(np.float64), side="left").astype(np.uint8)


def quantize_nf4(w: np.ndarray, blocksize: int = 64, nested: bool = True, blocksize2: int = 256) -> NF4State:
    """Blockwise NF4 quantiser over the row-major flattening of ``w`` (fp32 array)."""
    shape = tuple(w.shape)
    flat = np.ascontiguousarray(w, dtype=np.float32).reshape(-1)
    n = flat.size
    if n % blocksize or n % 2:
        raise ValueError("element count must be a multiple of the blocksize")
    blocks = flat.reshape(-1, blocksize)
    absmax = np.abs(blocks).max(axis=1).astype(np.float32)
    safe = np.where(absmax > 0, absmax, np.float32(1.0))
    idx = _nearest_code((blocks / safe[:, None]).reshape(-1), NF4_CODE)
    packed = ((idx[0::2] << 4) | idx[1::2]).astype(np.uint8)
    if not nested:
        return NF4State(packed, shape, blocksize, absmax, None, None, None, blocksize2)
    nb = absmax.size
    if nb % blocksize2:
        raise ValueError("number of blocks must be a multiple of the second-level blocksize")
    offset = np.asarray([absmax.mean(dtype=np.float64)], dtype=np.float32)
    centred = (absmax - offset[0]).reshape(-1, blocksize2)
    absmax2 = np.abs(centred).max(axis=1).astype(np.float32)
    safe2 = np.where(absmax2 > 0, absmax2, np.float32(1.0))
    code2 = dynamic_code_table()
    absq = _nearest_code((centred / safe2[:, None]).reshape(-1), code2)
    return NF4State(packed, shape, blocksize, absq, code2, absmax2, offset, blocksize2)
