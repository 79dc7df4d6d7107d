// Lossless 28-bit transfer format for 32-bit floating-point weights.
//
// A swap-in is bound by the host link, not by HBM or the CUs, so weights cross
// the link in fewer bytes and are expanded on the device.  The exponents of a
// weight tensor cluster: 15 consecutive exponent values cover all but a few
// values in ten thousand.  A word is therefore sent as sign + mantissa (24 bits)
// and a 4-bit exponent code relative to the tensor's window base; code 15 marks
// a word outside the window, whose full 32 bits travel in a side list and are
// patched in after expansion.  Any 32-bit pattern survives (zeros, denormals,
// infinities, NaNs, integers): the format is a statement about bits, not values.
//
// Layout of one group (8 words -> 28 bytes): bytes 0..23 hold eight 24-bit
// little-endian fields, (sign << 23) | mantissa; bytes 24..27 hold the eight
// 4-bit codes, word j in bits 4j..4j+3.  The last group of a tensor is padded
// with zero words.  64 words (256 B) become 224 B, so every 256-byte boundary
// of the expanded tensor is a group boundary of the packed one.
//
// The reference moves weights as they are (memory_manager.hpp:378-409); this
// has no counterpart there.
#pragma once
#include <cstdint>
#include <cstring>
#include <vector>

namespace tp {

constexpr uint32_t kPackWindow = 15;  // exponent codes 0..14; 15 = outside the window
constexpr uint32_t kPackEscape = 15;

inline uint64_t packed_bytes(uint64_t n_words) { return (n_words + 7) / 8 * 28; }

// The window base that leaves the fewest words outside, and that count.
inline void choose_window(const uint32_t* w, uint64_t n, uint32_t* base, uint64_t* outside) {
    uint64_t hist[256] = {0};
    for (uint64_t i = 0; i < n; ++i) hist[(w[i] >> 23) & 0xFF]++;
    uint64_t in = 0, best = 0;
    uint32_t best_base = 0;
    for (uint32_t e = 0; e < 256; ++e) {  // window [e - 14, e]
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

struct Escape {
    uint32_t index;  // word index, relative to whatever origin the caller adds
    uint32_t bits;
};

// Packs n words into packed_bytes(n) bytes at dst; words outside [base, base + 14] are appended to esc
// with index = origin + position.
inline void pack_words(const uint32_t* w, uint64_t n, uint32_t base, uint8_t* dst, uint64_t origin,
                       std::vector<Escape>* esc) {
    for (uint64_t g = 0; g * 8 < n; ++g) {
        uint8_t* o = dst + g * 28;
        uint32_t codes = 0;
        for (uint32_t j = 0; j < 8; ++j) {
            const uint64_t i = g * 8 + j;
            const uint32_t v = i < n ? w[i] : 0u;
            const uint32_t e = (v >> 23) & 0xFF;
            uint32_t code = kPackEscape;
            if (i >= n) {
                code = 0;
            } else if (e >= base && e - base < kPackWindow) {
                code = e - base;
            } else {
                esc->push_back({(uint32_t)(origin + i), v});
            }
            const uint32_t f = (v & 0x7FFFFFu) | ((v >> 31) << 23);
            o[3 * j] = (uint8_t)f;
            o[3 * j + 1] = (uint8_t)(f >> 8);
            o[3 * j + 2] = (uint8_t)(f >> 16);
            codes |= code << (4 * j);
        }
        std::memcpy(o + 24, &codes, 4);
    }
}

// Host-side expansion, the statement of what the device kernel must produce (escapes not applied).
inline void unpack_words(const uint8_t* src, uint64_t n, uint32_t base, uint32_t* out) {
    for (uint64_t i = 0; i < n; ++i) {
        const uint8_t* o = src + (i / 8) * 28;
        const uint32_t j = (uint32_t)(i % 8);
        const uint32_t f = (uint32_t)o[3 * j] | ((uint32_t)o[3 * j + 1] << 8) | ((uint32_t)o[3 * j + 2] << 16);
        uint32_t codes;
        std::memcpy(&codes, o + 24, 4);
        const uint32_t code = (codes >> (4 * j)) & 0xF;
        out[i] = (f & 0x7FFFFFu) | ((f >> 23) << 31) | (((base + code) & 0xFF) << 23);
    }
}

}  // namespace tp
