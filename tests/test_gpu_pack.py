"""The device kernel that expands the packed transfer format, on its own: arbitrary word counts
(partial last group, unit and block), partial ranges as a transfer group that ends inside a tensor
leaves them, and arbitrary contents, against the numpy statement of the format."""
import numpy as np
import pytest

from oracle import pack_ref
from torpor_amd import _lib

pytestmark = pytest.mark.gpu


def device_unpack(server, payload, n, base, ext, tab, w_from=0, w_to=None):
    L = _lib.lib()
    out = np.zeros(max(1, n), np.uint32)
    e = np.ascontiguousarray(ext, np.uint8)
    t = np.ascontiguousarray(tab, np.uint32)
    r = L.tp_unpack_words_device(server._h, np.ascontiguousarray(payload).ctypes.data, n, base,
                                 e.ctypes.data if len(e) else None, len(e), t.ctypes.data, w_from,
                                 n if w_to is None else w_to, out.ctypes.data)
    assert r == 0, r
    return out[:n]


def _cases(n, seed):
    rng = np.random.default_rng(seed)
    return [
        (rng.standard_normal(n) * 0.02).astype(np.float32).view(np.uint32),
        (rng.standard_normal(n) * np.exp(rng.uniform(-30, 30, n))).astype(np.float32).view(np.uint32),
        rng.integers(0, 1 << 32, n, dtype=np.uint64).astype(np.uint32),
        np.zeros(n, np.uint32),
    ]


@pytest.mark.parametrize("n", [1, 7, 8, 9, 63, 64, 65, 1000, 2047, 2048, 2049, 4099, 100003, 1 << 20])
def test_device_expansion_equals_the_format(gpu_server, n):
    for w in _cases(n, n):
        base, _ = pack_ref.best_window(w)
        payload, ext, tab = pack_ref.pack(w, base)
        assert np.array_equal(pack_ref.unpack(payload, n, base, ext), w)
        assert np.array_equal(device_unpack(gpu_server, payload, n, base, ext, tab), w)


@pytest.mark.parametrize("n,w_from,w_to", [(10000, 0, 64), (10000, 64, 2048), (10000, 1984, 2112), (10000, 2048, 10000),
                                           (10000, 4032, 9984), (100003, 65536, 100003), (100003, 12800, 12864)])
def test_partial_ranges_leave_the_rest_alone(gpu_server, n, w_from, w_to):
    """A transfer group that ends inside a tensor: only [w_from, w_to) is written, and the ranks in the
    extension stream are right although the block's earlier words belong to another group."""
    for w in _cases(n, n + w_from):
        base, _ = pack_ref.best_window(w)
        payload, ext, tab = pack_ref.pack(w, base)
        got = device_unpack(gpu_server, payload, n, base, ext, tab, w_from, w_to)
        want = np.full(n, 0xA5A5A5A5, np.uint32)
        want[w_from:w_to] = w[w_from:w_to]
        assert np.array_equal(got, want)


def test_device_expansion_checks_its_arguments(gpu_server):
    L = _lib.lib()
    w = np.zeros(128, np.uint32)
    payload = np.zeros(432, np.uint8)
    tab = np.zeros(1, np.uint32)
    h = gpu_server._h
    assert L.tp_unpack_words_device(h, payload.ctypes.data, 128, 300, None, 0, tab.ctypes.data, 0, 128, w.ctypes.data) == -22
    assert L.tp_unpack_words_device(h, payload.ctypes.data, 128, 0, None, 0, tab.ctypes.data, 8, 128, w.ctypes.data) == -22
    assert L.tp_unpack_words_device(h, payload.ctypes.data, 128, 0, None, 0, tab.ctypes.data, 0, 100, w.ctypes.data) == -22
    assert L.tp_unpack_words_device(h, payload.ctypes.data, 128, 0, None, 0, tab.ctypes.data, 64, 129, w.ctypes.data) == -22
    payload[192] = 7    # first word asks for an extension byte that is not there
    assert L.tp_unpack_words_device(h, payload.ctypes.data, 128, 0, None, 0, tab.ctypes.data, 0, 128, w.ctypes.data) == -22
