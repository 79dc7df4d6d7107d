"""The device kernels that expand the 28-bit transfer format, on their own: arbitrary word counts
(partial last group, partial last workgroup) and contents against the numpy statement of the format."""
import ctypes as C

import numpy as np
import pytest

from oracle import pack_ref
from torpor_amd import _lib

pytestmark = pytest.mark.gpu


def device_unpack(server, packed, n, base, pairs):
    L = _lib.lib()
    out = np.zeros(max(1, n), np.uint32)
    p = np.ascontiguousarray(pairs, np.uint32)
    r = L.tp_unpack_words_device(server._h, np.ascontiguousarray(packed).ctypes.data, n, base,
                                 p.ctypes.data if len(p) else None, len(p), out.ctypes.data)
    assert r == 0, r
    return out[:n]


@pytest.mark.parametrize("n", [1, 7, 8, 9, 63, 64, 65, 1000, 2047, 2048, 2049, 4099, 100003, 1 << 20])
def test_device_expansion_equals_the_format(gpu_server, n):
    rng = np.random.default_rng(n)
    cases = [
        (rng.standard_normal(n) * 0.02).astype(np.float32).view(np.uint32),
        (rng.standard_normal(n) * np.exp(rng.uniform(-30, 30, n))).astype(np.float32).view(np.uint32),
        rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32),
        np.zeros(n, np.uint32),
    ]
    for w in cases:
        base, _ = pack_ref.best_window(w)
        packed, pairs = pack_ref.pack(w, base)
        assert np.array_equal(pack_ref.unpack(packed, n, base, pairs), w)
        assert np.array_equal(device_unpack(gpu_server, packed, n, base, pairs), w)


def test_device_expansion_checks_its_arguments(gpu_server):
    L = _lib.lib()
    w = np.zeros(8, np.uint32)
    packed = np.zeros(28, np.uint8)
    bad = np.array([[8, 1]], np.uint32)
    assert L.tp_unpack_words_device(gpu_server._h, packed.ctypes.data, 8, 0, bad.ctypes.data, 1, w.ctypes.data) == -22
    assert L.tp_unpack_words_device(gpu_server._h, packed.ctypes.data, 8, 300, None, 0, w.ctypes.data) == -22
    big = 1 << 26   # 256 MiB of words: more than the workspace holds
    assert L.tp_unpack_words_device(gpu_server._h, packed.ctypes.data, big, 0, None, 0, w.ctypes.data) == -22
