// Lossless transfer format for 32-bit floating-point weights: 27 bits per word plus one byte for
// the few words outside their tensor's exponent window.
//
// A swap-in is bound by the host link, not by HBM or the CUs, so weights cross the link in fewer
// bytes and are expanded on the device.  The exponents of a weight tensor cluster: 7 consecutive
// exponent values hold about 97 % of the words of an initialised or trained tensor (their entropy
// is about 2.5 bits).  A word is sent as sign + mantissa (24 bits) and a 3-bit exponent code
// relative to the tensor's window base; code 7 marks a word outside the window, whose exponent
// byte travels in the tensor's extension stream, in word order.  Any 32-bit pattern survives
// (zeros, denormals, infinities, NaNs, integers): the format is a statement about bits.
//
// Payload: units of 64 words (256 bytes of the tensor) -> 216 bytes: eight groups of eight 24-bit
// little-endian fields, (sign << 23) | mantissa, then 24 bytes of codes, group g of the unit in
// bits 24g .. 24g+23, word j of the group in bits 3j .. 3j+2 of those.  The last unit is padded
// with zero words (code 0, no extension byte).  Every 256-byte boundary of the tensor is a unit
// boundary of the payload, so a transfer group that ends inside a tensor ends between units.
//
// Block table: the device expands blocks of 2048 words (32 units) independently; entry b is the
// number of extension bytes that belong to the words before block b.
//
// The reference moves weights as they are (memory_manager.hpp:378-409); this has no counterpart
// there.
#pragma once
#include <cstdint>
#include <cstring>
#include <vector>

namespace tp {

constexpr uint32_t kPackWindow = 7;      // exponent codes 0..6
constexpr uint32_t kPackExtended = 7;    // exponent in the extension stream
constexpr uint64_t kPackUnitWords = 64;  // 256 B of tensor -> 216 B of payload
constexpr uint64_t kPackUnitBytes = 216;
constexpr uint64_t kPackBlockWords = 2048;

inline uint64_t packed_bytes(uint64_t n_words) { return (n_words + kPackUnitWords - 1) / kPackUnitWords * kPackUnitBytes; }
inline uint64_t packed_blocks(uint64_t n_words) { return (n_words + kPackBlockWords - 1) / kPackBlockWords; }

// The window base that leaves the fewest words outside, and that count.
inline void choose_window(const uint32_t* w, uint64_t n, uint32_t* base, uint64_t* outside) {
    uint64_t hist[256] = {0};
    for (uint64_t i = 0; i < n; ++i) hist[(w[i] >> 23) & 0xFF]++;
    uint64_t in = 0, best = 0;
    uint32_t best_base = 0;
    for (uint32_t e = 0; e < 256; ++e) {  // window [e - 6, e]
        in += hist[e];
        if (e >= kPackWindow) in -= hist[e - kPackWindow];
        if (in > best) {
            best = in;
            best_base = e >= kPackWindow - 1 ? e - (kPackWindow - 1) : 0;
        }
    }
    *base = best_base;
    *outside = n - best;
}

// Packs n words: payload (packed_bytes(n), every byte of it written), extension bytes appended to ext,
// block_tab[packed_blocks(n)] filled with the extension count before each block.
inline void pack_words(const uint32_t* w, uint64_t n, uint32_t base, uint8_t* payload, std::vector<uint8_t>* ext,
                       uint32_t* block_tab) {
    const uint64_t ext0 = ext->size();
    for (uint64_t u = 0; u * kPackUnitWords < n; ++u) {
        uint8_t* o = payload + u * kPackUnitBytes;
        if (u % (kPackBlockWords / kPackUnitWords) == 0) block_tab[u / (kPackBlockWords / kPackUnitWords)] = (uint32_t)(ext->size() - ext0);
        for (uint32_t g = 0; g < 8; ++g) {
            uint32_t codes = 0;
            for (uint32_t j = 0; j < 8; ++j) {
                const uint64_t i = u * kPackUnitWords + g * 8 + j;
                const uint32_t v = i < n ? w[i] : 0u;
                const uint32_t e = (v >> 23) & 0xFF;
                uint32_t code = 0;
                if (i < n) {
                    if (e >= base && e - base < kPackWindow) {
                        code = e - base;
                    } else {
                        code = kPackExtended;
                        ext->push_back((uint8_t)e);
                    }
                }
                const uint32_t f = (v & 0x7FFFFFu) | ((v >> 31) << 23);
                uint8_t* fo = o + g * 24 + 3 * j;
                fo[0] = (uint8_t)f;
                fo[1] = (uint8_t)(f >> 8);
                fo[2] = (uint8_t)(f >> 16);
                codes |= code << (3 * j);
            }
            uint8_t* co = o + 192 + 3 * g;
            co[0] = (uint8_t)codes;
            co[1] = (uint8_t)(codes >> 8);
            co[2] = (uint8_t)(codes >> 16);
        }
    }
}

// Host-side expansion, the statement of what the device kernel must produce.  Returns the number
// of extension bytes consumed, or UINT64_MAX if the stream is too short.
inline uint64_t unpack_words(const uint8_t* payload, uint64_t n, uint32_t base, const uint8_t* ext, uint64_t n_ext,
                             uint32_t* out) {
    uint64_t used = 0;
    for (uint64_t i = 0; i < n; ++i) {
        const uint8_t* o = payload + (i / kPackUnitWords) * kPackUnitBytes;
        const uint32_t g = (uint32_t)(i % kPackUnitWords) / 8, j = (uint32_t)(i % 8);
        const uint8_t* fo = o + g * 24 + 3 * j;
        const uint32_t f = (uint32_t)fo[0] | ((uint32_t)fo[1] << 8) | ((uint32_t)fo[2] << 16);
        const uint8_t* co = o + 192 + 3 * g;
        const uint32_t codes = (uint32_t)co[0] | ((uint32_t)co[1] << 8) | ((uint32_t)co[2] << 16);
        const uint32_t code = (codes >> (3 * j)) & 7;
        uint32_t e = base + code;
        if (code == kPackExtended) {
            if (used >= n_ext) return UINT64_MAX;
            e = ext[used++];
        }
        out[i] = (f & 0x7FFFFFu) | ((f >> 23) << 31) | ((e & 0xFF) << 23);
    }
    return used;
}

}  // namespace tp
