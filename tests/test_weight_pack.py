"""The packed transfer format: the library's host packer against the numpy statement of the format,
a hand-worked unit, exhaustive sign x exponent coverage, brute-force window choice and the block
table.  (The device expansion is checked in tests/test_gpu_pack.py and, through whole swap-ins, in
tests/test_gpu_swap.py.)"""
import ctypes as C

import numpy as np
import pytest

from oracle import pack_ref
from torpor_amd import _lib


def lib_pack(words):
    L = _lib.lib()
    w = np.ascontiguousarray(words, np.uint32)
    payload = np.full(max(1, L.tp_pack_bound(len(w))), 0xEE, np.uint8)
    base, n_ext = C.c_int32(), C.c_uint64()
    ext = np.zeros(max(1, len(w)), np.uint8)
    tab = np.zeros(max(1, L.tp_pack_blocks(len(w))), np.uint32)
    r = L.tp_pack_words(w.ctypes.data, len(w), payload.ctypes.data, C.byref(base), ext.ctypes.data, len(ext),
                        C.byref(n_ext), tab.ctypes.data)
    assert r == 0
    return payload[:L.tp_pack_bound(len(w))], base.value, ext[:n_ext.value].copy(), tab[:L.tp_pack_blocks(len(w))]


def lib_unpack(payload, n, base, ext):
    L = _lib.lib()
    out = np.zeros(max(1, n), np.uint32)
    e = np.ascontiguousarray(ext, np.uint8)
    r = L.tp_unpack_words(np.ascontiguousarray(payload).ctypes.data, n, base, e.ctypes.data if len(e) else None, len(e),
                          out.ctypes.data)
    assert r == 0
    return out[:n]


def f32(*vals):
    return np.array(vals, np.float32).view(np.uint32)


def test_hand_worked_unit():
    """Eight words: 1.0 = 0x3F800000 (exponent 127, mantissa 0), -1.5 = 0xBFC00000 (sign, 127,
    0x400000), 0.5 (126), 2.0 (128), 0.0 (exponent 0: outside), then three more 1.0.  Seven of the
    eight have exponents 126..128; the scan keeps the first base that holds them, 128 - 6 = 122."""
    w = f32(1.0, -1.5, 0.5, 2.0, 0.0, 1.0, 1.0, 1.0)
    payload, base, ext, tab = lib_pack(w)
    assert base == 122 and ext.tolist() == [0] and tab.tolist() == [0]
    assert len(payload) == 216 == _lib.lib().tp_pack_bound(64) and _lib.lib().tp_pack_bound(65) == 432
    assert _lib.lib().tp_pack_blocks(2048) == 1 and _lib.lib().tp_pack_blocks(2049) == 2
    fields = [0x000000, 0xC00000, 0, 0, 0, 0, 0, 0]
    want = np.zeros(216, np.uint8)
    for j, f in enumerate(fields):
        want[3 * j:3 * j + 3] = [f & 0xFF, (f >> 8) & 0xFF, f >> 16]
    codes = [5, 5, 4, 6, 7, 5, 5, 5]
    word = sum(c << (3 * j) for j, c in enumerate(codes))
    want[192:195] = [word & 0xFF, (word >> 8) & 0xFF, word >> 16]
    assert np.array_equal(payload, want)
    assert np.array_equal(lib_unpack(payload, 8, base, ext), w)


def test_every_sign_and_exponent_survives():
    rng = np.random.default_rng(0)
    e = np.repeat(np.arange(256, dtype=np.uint32), 2)
    s = np.tile(np.array([0, 1], np.uint32), 256)
    for mant in (np.zeros(512, np.uint32), np.full(512, 0x7FFFFF, np.uint32), rng.integers(0, 1 << 23, 512).astype(np.uint32)):
        w = (s << 31) | (e << 23) | mant          # includes +-0, denormals, +-inf, NaNs
        payload, base, ext, tab = lib_pack(w)
        assert len(ext) == 512 - 14               # 7 exponents x 2 signs fit the window
        assert np.array_equal(lib_unpack(payload, len(w), base, ext), w)
        assert np.array_equal(pack_ref.unpack(payload, len(w), base, ext), w)


@pytest.mark.parametrize("n", [1, 7, 8, 9, 63, 64, 65, 1000, 2047, 2048, 2049, 4099, 10000])
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
        payload, base, ext, tab = lib_pack(w)
        rbase, routside = pack_ref.best_window(w)
        assert len(ext) == routside                        # the library's window is as good as the best
        rpayload, rext, rtab = pack_ref.pack(w, base)
        assert np.array_equal(payload, rpayload) and np.array_equal(ext, rext) and np.array_equal(tab, rtab)
        assert np.array_equal(lib_unpack(payload, n, base, ext), w)
        assert np.array_equal(pack_ref.unpack(rpayload, n, base, rext), w)


def test_block_table_counts_extension_bytes_before_each_block():
    rng = np.random.default_rng(3)
    w = (rng.standard_normal(5 * 2048 + 100) * np.exp(rng.uniform(-3, 3, 5 * 2048 + 100))).astype(np.float32).view(np.uint32)
    payload, base, ext, tab = lib_pack(w)
    e = (w >> 23) & 0xFF
    outside = (e < base) | (e >= base + 7)
    want = [int(outside[:b * 2048].sum()) for b in range(6)]
    assert tab.tolist() == want and len(ext) == int(outside.sum()) > 100


def test_initialised_weights_shrink_by_a_seventh():
    w = (np.random.default_rng(5).standard_normal(1 << 20) * 0.02).astype(np.float32).view(np.uint32)
    payload, base, ext, tab = lib_pack(w)
    assert len(payload) == len(w) * 27 // 8
    assert 0.015 * len(w) < len(ext) < 0.035 * len(w)   # a Gaussian leaves about 2.5 % outside seven binades
    assert len(payload) + len(ext) + 4 * len(tab) < 0.855 * 4 * len(w)


def test_argument_checks():
    L = _lib.lib()
    w = np.zeros(8, np.uint32)
    out = np.zeros(216, np.uint8)
    tab = np.zeros(1, np.uint32)
    base, n_ext = C.c_int32(), C.c_uint64()
    assert L.tp_pack_words(w.ctypes.data, 8, None, C.byref(base), None, 0, C.byref(n_ext), tab.ctypes.data) == -22
    # more extension bytes than room: refused, count reported
    assert L.tp_pack_words(f32(1, 0, 0, 0, 1e30, 1, 1, 1).ctypes.data, 8, out.ctypes.data, C.byref(base), None, 0,
                           C.byref(n_ext), tab.ctypes.data) == -12
    assert n_ext.value == 4
    # a stream shorter than the codes ask for, a base out of range
    assert L.tp_unpack_words(out.ctypes.data, 8, base.value, None, 0, w.ctypes.data) == -22
    assert L.tp_unpack_words(out.ctypes.data, 8, 256, None, 0, w.ctypes.data) == -22
