"""TEST INFRASTRUCTURE ONLY -- numpy statement of the packed transfer format for 32-bit weight words.

The reference has no such format (it sends weights as they are, include/server/memory_manager.hpp:378-409),
so there is nothing of the reference's to follow here; the format is pinned by what it must satisfy:
  * unpack(pack(x)) == x for every 32-bit pattern (checked exhaustively over sign x exponent and on
    random mantissas, zeros, denormals, infinities, NaNs), the one property the engine relies on;
  * a hand-worked unit (tests/test_weight_pack.py) fixes the byte layout;
  * the window choice is checked against brute force over all 256 bases;
  * the block table is checked against a running count.
Written with whole-array numpy operations, independently of the library's word-by-word C++ loop.
"""
import numpy as np

WINDOW = 7          # codes 0..6 are exponents base..base+6, code 7 = next byte of the extension stream
UNIT_WORDS, UNIT_BYTES, BLOCK_WORDS = 64, 216, 2048


def best_window(words):
    """(base, number of words outside [base, base+6]); the lowest base among the best."""
    e = (np.asarray(words, np.uint32) >> 23) & 0xFF
    hist = np.bincount(e, minlength=256)
    inside = [int(hist[b:b + WINDOW].sum()) for b in range(256)]
    base = int(np.argmax(inside))
    return base, int(len(e) - inside[base])


def pack(words, base):
    """-> (payload bytes, extension bytes, block table) for window base `base`."""
    w = np.asarray(words, np.uint32)
    n = len(w)
    units = (n + UNIT_WORDS - 1) // UNIT_WORDS
    padded = np.zeros(units * UNIT_WORDS, np.uint32)
    padded[:n] = w
    e = ((padded >> 23) & 0xFF).astype(np.int64)
    code = e - base
    outside = (code < 0) | (code >= WINDOW)
    outside[n:] = False
    code = np.where(outside, 7, code).astype(np.uint32)
    code[n:] = 0
    field = (padded & 0x7FFFFF) | ((padded >> 31) << 23)
    out = np.zeros((units, UNIT_BYTES), np.uint8)
    f = field.reshape(units, 8, 8)
    c = code.reshape(units, 8, 8)
    for g in range(8):
        for j in range(8):
            for k in range(3):
                out[:, g * 24 + 3 * j + k] = (f[:, g, j] >> (8 * k)) & 0xFF
        codes = np.zeros(units, np.uint32)
        for j in range(8):
            codes |= c[:, g, j] << np.uint32(3 * j)
        for k in range(3):
            out[:, 192 + 3 * g + k] = (codes >> (8 * k)) & 0xFF
    ext = e[outside].astype(np.uint8)
    before = np.concatenate([[0], np.cumsum(outside)])
    tab = before[np.arange(0, n, BLOCK_WORDS)].astype(np.uint32) if n else np.zeros(0, np.uint32)
    return out.reshape(-1), ext, tab


def unpack(payload, n, base, ext):
    u = np.asarray(payload, np.uint8).reshape(-1, UNIT_BYTES)
    fb = u[:, :192].reshape(-1, 8, 8, 3).astype(np.uint32)
    field = fb[..., 0] | (fb[..., 1] << 8) | (fb[..., 2] << 16)
    cb = u[:, 192:].reshape(-1, 8, 3).astype(np.uint32)
    codes = cb[..., 0] | (cb[..., 1] << 8) | (cb[..., 2] << 16)
    code = np.stack([(codes >> np.uint32(3 * j)) & 7 for j in range(8)], axis=2)
    field = field.reshape(-1)[:n]
    code = code.reshape(-1)[:n]
    e = (np.uint32(base) + code) & 0xFF
    is_ext = code == 7
    assert int(is_ext.sum()) == len(ext)
    e[is_ext] = np.asarray(ext, np.uint32)
    return ((field & 0x7FFFFF) | ((field >> 23) << 31) | (e << 23)).astype(np.uint32)
