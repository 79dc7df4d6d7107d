"""TEST INFRASTRUCTURE ONLY -- numpy statement of the 28-bit transfer format for 32-bit weight words.

The reference has no such format (it sends weights as they are, include/server/memory_manager.hpp:378-409),
so there is nothing of the reference's to follow here; the format is pinned by what it must satisfy:
  * unpack(pack(x)) == x for every 32-bit pattern (checked exhaustively over sign x exponent and on
    random mantissas, zeros, denormals, infinities, NaNs), the one property the engine relies on;
  * a hand-worked group (tests/test_weight_pack.py) fixes the byte layout;
  * the window choice is checked against brute force over all 256 bases.
Written with whole-array numpy operations, independently of the library's word-by-word C++ loop.
"""
import numpy as np

WINDOW = 15   # codes 0..14 are exponents base..base+14, code 15 marks a word listed separately


def best_window(words):
    """(base, number of words outside [base, base+14]); the lowest base among the best."""
    e = (np.asarray(words, np.uint32) >> 23) & 0xFF
    hist = np.bincount(e, minlength=256)
    inside = [int(hist[b:b + WINDOW].sum()) for b in range(256)]
    base = int(np.argmax(inside))
    return base, int(len(e) - inside[base])


def pack(words, base):
    """-> (packed bytes, pairs[(index, bits)]) for window base `base`."""
    w = np.asarray(words, np.uint32)
    n = len(w)
    groups = (n + 7) // 8
    padded = np.zeros(groups * 8, np.uint32)
    padded[:n] = w
    e = ((padded >> 23) & 0xFF).astype(np.int64)
    code = e - base
    outside = (code < 0) | (code >= WINDOW)
    outside[n:] = False
    code = np.where(outside, 15, code).astype(np.uint32)
    code[n:] = 0
    field = (padded & 0x7FFFFF) | ((padded >> 31) << 23)
    out = np.zeros((groups, 28), np.uint8)
    f = field.reshape(groups, 8)
    for j in range(8):
        out[:, 3 * j] = f[:, j] & 0xFF
        out[:, 3 * j + 1] = (f[:, j] >> 8) & 0xFF
        out[:, 3 * j + 2] = (f[:, j] >> 16) & 0xFF
    c = code.reshape(groups, 8)
    codes = np.zeros(groups, np.uint32)
    for j in range(8):
        codes |= c[:, j] << np.uint32(4 * j)
    out[:, 24:28] = codes.astype("<u4").view(np.uint8).reshape(groups, 4)
    idx = np.nonzero(outside)[0].astype(np.uint32)
    pairs = np.stack([idx, padded[idx]], axis=1).astype(np.uint32) if len(idx) else np.zeros((0, 2), np.uint32)
    return out.reshape(-1), pairs


def unpack(packed, n, base, pairs):
    g = np.asarray(packed, np.uint8).reshape(-1, 28)
    b = g[:, :24].reshape(-1, 8, 3).astype(np.uint32)
    field = b[:, :, 0] | (b[:, :, 1] << 8) | (b[:, :, 2] << 16)
    codes = g[:, 24:28].copy().view("<u4").reshape(-1)
    code = np.stack([(codes >> np.uint32(4 * j)) & 0xF for j in range(8)], axis=1)
    w = (field & 0x7FFFFF) | ((field >> 23) << 31) | (((np.uint32(base) + code) & 0xFF) << 23)
    w = w.reshape(-1)[:n].astype(np.uint32)
    for i, bits in np.asarray(pairs, np.uint32).reshape(-1, 2):
        w[i] = bits
    return w
