// Minimal read-only access to FlatBuffers data (little endian hosts only).
// Enough for common/dab.fbs of the reference: tables, strings, vectors of
// scalars / strings / tables.  The flatbuffers library is not a dependency.
//
// Every access is checked against the extent of the buffer the table came
// from: an offset, vtable, string or vector that leaves [base, base + size)
// throws std::invalid_argument, so a truncated or corrupt model is an error
// and never a read outside the caller's memory.
#pragma once

#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace fb {

[[noreturn]] inline void malformed(const char *what) {
    throw std::invalid_argument(std::string("malformed model buffer: ") + what);
}

// The buffer a table lives in.
struct Span {
    const uint8_t *base = nullptr;
    size_t size = 0;
    // [q, q + n) inside the buffer?
    bool holds(const uint8_t *q, size_t n) const {
        return q >= base && (size_t)(q - base) <= size && n <= size - (size_t)(q - base);
    }
    void need(const uint8_t *q, size_t n, const char *what) const {
        if (!holds(q, n)) malformed(what);
    }
    template <class T>
    T load(const uint8_t *q, const char *what) const {
        need(q, sizeof(T), what);
        T v;
        std::memcpy(&v, q, sizeof(T));
        return v;
    }
    // q + off, refusing pointers that would leave the buffer (also by wrapping around)
    const uint8_t *advance(const uint8_t *q, uint64_t off, const char *what) const {
        if (!holds(q, 0) || off > size - (size_t)(q - base)) malformed(what);
        return q + off;
    }
};

// A table position inside a buffer; `slot` is the 0-based declaration index of a field.
struct Table {
    Span buf;
    const uint8_t *p = nullptr;
    bool valid() const { return p != nullptr; }

    uint16_t field_offset(int slot) const {
        const int32_t back = buf.load<int32_t>(p, "table header");
        // the vtable sits `back` bytes before the table (after it when negative)
        const int64_t vt_pos = (int64_t)(p - buf.base) - back;
        if (vt_pos < 0 || (uint64_t)vt_pos > buf.size) malformed("vtable offset");
        const uint8_t *vt = buf.base + vt_pos;
        const uint16_t vt_size = buf.load<uint16_t>(vt, "vtable size");
        if (vt_size < 4 || (vt_size & 1)) malformed("vtable size");
        buf.need(vt, vt_size, "vtable");
        const int o = 4 + 2 * slot;
        if (o + 2 > vt_size) return 0;
        const uint16_t f = buf.load<uint16_t>(vt + o, "vtable entry");
        if (f != 0) {
            const uint16_t table_size = buf.load<uint16_t>(vt + 2, "vtable table size");
            if (f < 4 || f >= table_size) malformed("field offset outside its table");
        }
        return f;
    }
    template <class T>
    T scalar(int slot, T def) const {
        const uint16_t f = field_offset(slot);
        return f ? buf.load<T>(p + f, "scalar field") : def;
    }
    const uint8_t *indirect(int slot) const {
        const uint16_t f = field_offset(slot);
        if (!f) return nullptr;
        const uint8_t *q = p + f;
        return buf.advance(q, buf.load<uint32_t>(q, "offset field"), "offset field target");
    }
    bool has(int slot) const { return field_offset(slot) != 0; }
    std::string str_at(const uint8_t *q) const {
        const uint32_t len = buf.load<uint32_t>(q, "string length");
        buf.need(q + 4, len, "string");
        return std::string(reinterpret_cast<const char *>(q + 4), len);
    }
    std::string str(int slot) const {
        const uint8_t *q = indirect(slot);
        return q ? str_at(q) : std::string();
    }
    Table table_at(const uint8_t *q) const {
        Table t;
        t.buf = buf;
        t.p = q;
        buf.need(q, 4, "table");
        return t;
    }
    Table table(int slot) const {
        const uint8_t *q = indirect(slot);
        return q ? table_at(q) : Table();
    }
    // vector of scalars: pointer to the first element and the element count (the whole vector lies in the buffer)
    template <class T>
    const T *vec(int slot, uint32_t *count) const {
        const uint8_t *q = indirect(slot);
        if (!q) {
            *count = 0;
            return nullptr;
        }
        const uint32_t n = buf.load<uint32_t>(q, "vector length");
        if ((uint64_t)n * sizeof(T) > buf.size) malformed("vector longer than the buffer");
        buf.need(q + 4, (size_t)n * sizeof(T), "vector");
        *count = n;
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
    // vectors of offsets (tables, strings)
    uint32_t vec_len(int slot) const {
        uint32_t n = 0;
        (void)vec<uint32_t>(slot, &n);
        return n;
    }
    const uint8_t *vec_elem(int slot, uint32_t i) const {
        uint32_t n = 0;
        const uint32_t *d = vec<uint32_t>(slot, &n);
        if (i >= n) malformed("vector index");
        const uint8_t *q = reinterpret_cast<const uint8_t *>(d) + 4 * (size_t)i;
        return buf.advance(q, buf.load<uint32_t>(q, "vector element"), "vector element target");
    }
    Table vec_table(int slot, uint32_t i) const { return table_at(vec_elem(slot, i)); }
    std::string vec_str(int slot, uint32_t i) const { return str_at(vec_elem(slot, i)); }
};

inline Table root(const void *data, size_t size) {
    Table t;
    t.buf.base = static_cast<const uint8_t *>(data);
    t.buf.size = size;
    if (data == nullptr || size < 8) malformed("shorter than a FlatBuffers header");
    const uint8_t *q = t.buf.advance(t.buf.base, t.buf.load<uint32_t>(t.buf.base, "root offset"), "root table");
    t.buf.need(q, 4, "root table");
    t.p = q;
    return t;
}

}  // namespace fb
