"""The 28-bit transfer format: the library's host packer against the numpy statement of the format,
a hand-worked group, exhaustive sign x exponent coverage and brute-force window choice.  (The device
expansion is checked against the same property, bit-identical weights after a swap-in, in
tests/test_gpu_swap.py.)"""
import ctypes as C

import numpy as np
import pytest

from oracle import pack_ref
from torpor_amd import _lib


def lib_pack(words):
    L = _lib.lib()
    w = np.ascontiguousarray(words, np.uint32)
    out = np.zeros(L.tp_pack_bound(len(w)), np.uint8)
    base, n_pairs = C.c_int32(), C.c_uint64()
    pairs = np.zeros((max(1, len(w)), 2), np.uint32)
    r = L.tp_pack_words(w.ctypes.data, len(w), out.ctypes.data, C.byref(base), pairs.ctypes.data, len(pairs), C.byref(n_pairs))
    assert r == 0
    return out, base.value, pairs[:n_pairs.value].copy()


def lib_unpack(packed, n, base, pairs):
    L = _lib.lib()
    out = np.zeros(max(1, n), np.uint32)
    p = np.ascontiguousarray(pairs, np.uint32)
    r = L.tp_unpack_words(np.ascontiguousarray(packed).ctypes.data, n, base, p.ctypes.data if len(p) else None, len(p), out.ctypes.data)
    assert r == 0
    return out[:n]


def f32(*vals):
    return np.array(vals, np.float32).view(np.uint32)


def test_hand_worked_group():
    """1.0 = 0x3F800000 (exponent 127, mantissa 0), -1.5 = 0xBFC00000 (sign, 127, 0x400000),
    0.5 (126), 2.0 (128), 0.0 (exponent 0: outside), then three more 1.0.  Window [126, 140] holds
    seven of the eight, as does any base from 114 to 126; the scan keeps the first best, base 114."""
    w = f32(1.0, -1.5, 0.5, 2.0, 0.0, 1.0, 1.0, 1.0)
    packed, base, pairs = lib_pack(w)
    assert base == 114 and pairs.tolist() == [[4, 0]]
    fields = [0x000000, 0xC00000, 0x000000, 0x000000, 0x000000, 0x000000, 0x000000, 0x000000]
    codes = [13, 13, 12, 14, 15, 13, 13, 13]
    want = []
    for f in fields:
        want += [f & 0xFF, (f >> 8) & 0xFF, f >> 16]
    word = sum(c << (4 * j) for j, c in enumerate(codes))
    want += [(word >> (8 * k)) & 0xFF for k in range(4)]
    assert packed.tolist() == want
    assert len(packed) == 28 == _lib.lib().tp_pack_bound(8) and _lib.lib().tp_pack_bound(9) == 56
    assert np.array_equal(lib_unpack(packed, 8, base, pairs), w)


def test_every_sign_and_exponent_survives():
    rng = np.random.default_rng(0)
    e = np.repeat(np.arange(256, dtype=np.uint32), 2)
    s = np.tile(np.array([0, 1], np.uint32), 256)
    for mant in (np.zeros(512, np.uint32), np.full(512, 0x7FFFFF, np.uint32), rng.integers(0, 1 << 23, 512).astype(np.uint32)):
        w = (s << 31) | (e << 23) | mant          # includes +-0, denormals, +-inf, NaNs
        packed, base, pairs = lib_pack(w)
        assert len(pairs) == 512 - 30             # 15 exponents x 2 signs fit the window
        assert np.array_equal(lib_unpack(packed, len(w), base, pairs), w)
        assert np.array_equal(pack_ref.unpack(packed, len(w), base, pairs), w)


@pytest.mark.parametrize("n", [1, 7, 8, 9, 63, 64, 65, 1000, 4099])
def test_library_and_numpy_agree_on_weight_like_and_arbitrary_words(n):
    rng = np.random.default_rng(n)
    cases = [
        (rng.standard_normal(n) * 0.02).astype(np.float32).view(np.uint32),        # initialised weights
        (rng.standard_normal(n) * np.exp(rng.uniform(-30, 30, n))).astype(np.float32).view(np.uint32),
        rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32),            # arbitrary bits
        np.zeros(n, np.uint32),
        np.full(n, 0x7FC00000, np.uint32),                                          # NaN
    ]
    for w in cases:
        packed, base, pairs = lib_pack(w)
        rbase, routside = pack_ref.best_window(w)
        assert len(pairs) == routside                      # the library's window is as good as the best
        rpacked, rpairs = pack_ref.pack(w, base)
        assert np.array_equal(packed, rpacked) and np.array_equal(pairs, rpairs)
        assert np.array_equal(lib_unpack(packed, n, base, pairs), w)
        assert np.array_equal(pack_ref.unpack(rpacked, n, base, rpairs), w)


def test_initialised_weights_shrink_by_an_eighth():
    w = (np.random.default_rng(5).standard_normal(1 << 20) * 0.02).astype(np.float32).view(np.uint32)
    packed, base, pairs = lib_pack(w)
    assert len(packed) == len(w) * 28 // 8
    assert len(pairs) < 4e-4 * len(w)     # |x| < 2^-14 of the largest binade: a few words in ten thousand
    assert len(packed) + 8 * len(pairs) < 0.88 * 4 * len(w)


def test_argument_checks():
    L = _lib.lib()
    w = np.zeros(8, np.uint32)
    out = np.zeros(28, np.uint8)
    base, n_pairs = C.c_int32(), C.c_uint64()
    assert L.tp_pack_words(w.ctypes.data, 8, None, C.byref(base), None, 0, C.byref(n_pairs)) == -22
    # more pairs than room: refused, count reported
    assert L.tp_pack_words(f32(1, 0, 0, 0, 1e30, 1, 1, 1).ctypes.data, 8, out.ctypes.data, C.byref(base), None, 0, C.byref(n_pairs)) == -12
    assert n_pairs.value == 4
    bad = np.array([[9, 1]], np.uint32)
    assert L.tp_unpack_words(out.ctypes.data, 8, 0, bad.ctypes.data, 1, w.ctypes.data) == -22
    assert L.tp_unpack_words(out.ctypes.data, 8, 256, None, 0, w.ctypes.data) == -22
