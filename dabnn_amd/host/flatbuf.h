// Minimal read-only access to FlatBuffers data (little endian hosts only).
// Enough for common/dab.fbs of the reference: tables, strings, vectors of
// scalars / strings / tables.  The flatbuffers library is not a dependency.
#pragma once

#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace fb {

template <class T>
inline T load(const uint8_t *p) {
    T v;
    std::memcpy(&v, p, sizeof(T));
    return v;
}

// A table position inside a buffer; `slot` is the 0-based declaration index of a field.
struct Table {
    const uint8_t *p = nullptr;
    bool valid() const { return p != nullptr; }
    uint16_t field_offset(int slot) const {
        const uint8_t *vt = p - load<int32_t>(p);
        const uint16_t vt_size = load<uint16_t>(vt);
        const int o = 4 + 2 * slot;
        return o < vt_size ? load<uint16_t>(vt + o) : 0;
    }
    template <class T>
    T scalar(int slot, T def) const {
        const uint16_t f = field_offset(slot);
        return f ? load<T>(p + f) : def;
    }
    const uint8_t *indirect(int slot) const {
        const uint16_t f = field_offset(slot);
        if (!f) return nullptr;
        const uint8_t *q = p + f;
        return q + load<uint32_t>(q);
    }
    bool has(int slot) const { return field_offset(slot) != 0; }
    std::string str(int slot) const {
        const uint8_t *q = indirect(slot);
        if (!q) return std::string();
        return std::string(reinterpret_cast<const char *>(q + 4), load<uint32_t>(q));
    }
    Table table(int slot) const {
        Table t;
        t.p = indirect(slot);
        return t;
    }
    // vector of scalars: pointer to the first element and the element count
    template <class T>
    const T *vec(int slot, uint32_t *count) const {
        const uint8_t *q = indirect(slot);
        if (!q) {
            *count = 0;
            return nullptr;
        }
        *count = load<uint32_t>(q);
        return reinterpret_cast<const T *>(q + 4);
    }
    template <class T>
    std::vector<T> vec_copy(int slot) const {
        uint32_t n = 0;
        const T *d = vec<T>(slot, &n);
        std::vector<T> out(n);
        if (n) std::memcpy(out.data(), d, n * sizeof(T));
        return out;
    }
    uint32_t vec_len(int slot) const {
        const uint8_t *q = indirect(slot);
        return q ? load<uint32_t>(q) : 0;
    }
    Table vec_table(int slot, uint32_t i) const {
        const uint8_t *q = indirect(slot) + 4 + 4 * i;
        Table t;
        t.p = q + load<uint32_t>(q);
        return t;
    }
    std::string vec_str(int slot, uint32_t i) const {
        const uint8_t *q = indirect(slot) + 4 + 4 * i;
        const uint8_t *s = q + load<uint32_t>(q);
        return std::string(reinterpret_cast<const char *>(s + 4), load<uint32_t>(s));
    }
};

inline Table root(const void *buf) {
    const uint8_t *b = static_cast<const uint8_t *>(buf);
    Table t;
    t.p = b + load<uint32_t>(b);
    return t;
}

}  // namespace fb
