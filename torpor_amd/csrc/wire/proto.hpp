// Minimal proto3 wire codec (varint keys, length-delimited, fixed32/64), enough for the
// reference's signal.proto and for the op messages of the data plane.  protoc and the
// protobuf C++ runtime are not part of the ROCm image, so the messages are written and
// parsed by hand from the encoding specification; proto3 rules apply (scalar fields equal
// to their default are not emitted, unknown fields are skipped on read, a negative int32 is
// a 10-byte varint).
#pragma once
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace pb {

enum WireType : int { WT_VARINT = 0, WT_FIXED64 = 1, WT_LEN = 2, WT_FIXED32 = 5 };

class Writer {
public:
    std::string out;
    void varint(uint64_t v) {
        while (v >= 0x80) {
            out.push_back((char)((v & 0x7F) | 0x80));
            v >>= 7;
        }
        out.push_back((char)v);
    }
    void key(int field, int wt) { varint(((uint64_t)field << 3) | (uint64_t)wt); }
    void u64(int field, uint64_t v) {
        if (!v) return;
        key(field, WT_VARINT);
        varint(v);
    }
    void i64(int field, int64_t v) { u64(field, (uint64_t)v); }
    void i32(int field, int32_t v) { u64(field, (uint64_t)(int64_t)v); }  // sign-extended, as protobuf does
    void boolean(int field, bool v) { u64(field, v ? 1 : 0); }
    void f32(int field, float v) {
        uint32_t b;
        std::memcpy(&b, &v, 4);
        if (!b) return;
        key(field, WT_FIXED32);
        out.append(reinterpret_cast<const char*>(&b), 4);  // little endian host
    }
    void f64(int field, double v) {
        uint64_t b;
        std::memcpy(&b, &v, 8);
        if (!b) return;
        key(field, WT_FIXED64);
        out.append(reinterpret_cast<const char*>(&b), 8);
    }
    void bytes(int field, const void* data, size_t len) {
        if (!len) return;
        key(field, WT_LEN);
        varint(len);
        out.append(static_cast<const char*>(data), len);
    }
    void str(int field, const std::string& s) { bytes(field, s.data(), s.size()); }
    // embedded message / repeated element: emitted even when empty
    void message(int field, const std::string& body) {
        key(field, WT_LEN);
        varint(body.size());
        out.append(body);
    }
    void packed_u64(int field, const std::vector<uint64_t>& v) {
        if (v.empty()) return;
        Writer w;
        for (uint64_t x : v) w.varint(x);
        message(field, w.out);
    }
    void packed_i64(int field, const std::vector<int64_t>& v) {
        if (v.empty()) return;
        Writer w;
        for (int64_t x : v) w.varint((uint64_t)x);
        message(field, w.out);
    }
    void packed_f32(int field, const std::vector<float>& v) {
        if (v.empty()) return;
        key(field, WT_LEN);
        varint(v.size() * 4);
        out.append(reinterpret_cast<const char*>(v.data()), v.size() * 4);
    }
};

struct View {
    const uint8_t* p = nullptr;
    size_t n = 0;
    std::string str() const { return std::string(reinterpret_cast<const char*>(p), n); }
};

class Reader {
public:
    Reader(const void* data, size_t len) : p_(static_cast<const uint8_t*>(data)), end_(p_ + len) {}
    explicit Reader(const View& v) : p_(v.p), end_(v.p + v.n) {}
    bool ok() const { return ok_; }
    bool done() const { return p_ >= end_ || !ok_; }

    // Reads the next key; false at the end of the buffer or on malformed input.
    bool next(int* field, int* wt) {
        if (done()) return false;
        uint64_t k = varint();
        if (!ok_) return false;
        *field = (int)(k >> 3);
        *wt = (int)(k & 7);
        if (*field == 0) ok_ = false;
        return ok_;
    }
    uint64_t varint() {
        uint64_t v = 0;
        for (int shift = 0; shift < 70; shift += 7) {
            if (p_ >= end_) {
                ok_ = false;
                return 0;
            }
            const uint8_t b = *p_++;
            if (shift < 64) v |= (uint64_t)(b & 0x7F) << shift;
            if (!(b & 0x80)) return v;
        }
        ok_ = false;
        return 0;
    }
    float f32() {
        float v = 0;
        if (end_ - p_ < 4) {
            ok_ = false;
            return 0;
        }
        std::memcpy(&v, p_, 4);
        p_ += 4;
        return v;
    }
    double f64() {
        double v = 0;
        if (end_ - p_ < 8) {
            ok_ = false;
            return 0;
        }
        std::memcpy(&v, p_, 8);
        p_ += 8;
        return v;
    }
    View bytes() {
        View v;
        const uint64_t n = varint();
        if (!ok_ || n > (uint64_t)(end_ - p_)) {
            ok_ = false;
            return v;
        }
        v.p = p_;
        v.n = (size_t)n;
        p_ += n;
        return v;
    }
    void skip(int wt) {
        switch (wt) {
            case WT_VARINT: (void)varint(); break;
            case WT_FIXED64: (void)f64(); break;
            case WT_LEN: (void)bytes(); break;
            case WT_FIXED32: (void)f32(); break;
            default: ok_ = false; break;
        }
    }
    // scalar numeric field that may arrive as varint (normal) - other wire types are skipped
    bool read_u64(int wt, uint64_t* v) {
        if (wt != WT_VARINT) {
            skip(wt);
            return false;
        }
        *v = varint();
        return ok_;
    }
    // repeated numeric field: accepts packed and unpacked encodings
    void read_rep_varint(int wt, std::vector<uint64_t>* out) {
        if (wt == WT_LEN) {
            Reader r(bytes());
            while (!r.done()) out->push_back(r.varint());
            if (!r.ok()) ok_ = false;
        } else if (wt == WT_VARINT) {
            out->push_back(varint());
        } else {
            skip(wt);
        }
    }
    void read_rep_f32(int wt, std::vector<float>* out) {
        if (wt == WT_LEN) {
            Reader r(bytes());
            while (!r.done()) out->push_back(r.f32());
            if (!r.ok()) ok_ = false;
        } else if (wt == WT_FIXED32) {
            out->push_back(f32());
        } else {
            skip(wt);
        }
    }

private:
    const uint8_t* p_;
    const uint8_t* end_;
    bool ok_ = true;
};

}  // namespace pb
