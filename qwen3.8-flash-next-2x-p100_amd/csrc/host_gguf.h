// Read-only access to GGUF model files for the tensors of this path: a layer's routed and shared IQ3_S experts and its
// router rows (the reference's reader: gguf.hpp:25-45, gguf.cpp:219-320; its slicing of expert tensors into the layouts
// the operators read: model.cpp:702-741 expert_rows2, 768-790 expert_cols, 988-989 the router's rows).
//
// Host code only. A file (and the "-0000N-of-0000M" shards beside it) is mapped, never copied; a header that does not
// add up is refused with a message that names the tensor, as the reference's reader refuses it (tools/gguf_test.cpp).
// Tensors of other quantisations can be found and described, but only F32 / BF16 router rows and IQ3_S experts are turned
// into a layer here; the reference's load-time re-quantisation of a file's other tensors is not part of this path.
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/fnx_mi355x.h"

namespace fnx {
namespace gguf {

struct BlockShape {
    int values, bytes;
};
// ggml's block shapes by type id (the public ggml type table; the ids the reference names: gguf.hpp:22-27)
inline bool block_shape(uint32_t type, BlockShape& b) {
    static const struct {
        uint32_t id;
        BlockShape s;
    } table[] = {{0, {1, 4}},     {1, {1, 2}},      {2, {32, 18}},    {3, {32, 20}},    {6, {32, 22}},    {7, {32, 24}},    {8, {32, 34}},
                 {9, {32, 36}},   {10, {256, 84}},  {11, {256, 110}}, {12, {256, 144}}, {13, {256, 176}}, {14, {256, 210}}, {15, {256, 292}},
                 {16, {256, 66}}, {17, {256, 74}},  {18, {256, 98}},  {19, {256, 50}},  {20, {32, 18}},   {21, {256, 110}}, {22, {256, 82}},
                 {23, {256, 136}}, {24, {1, 1}},    {25, {1, 2}},     {26, {1, 4}},     {27, {1, 8}},     {28, {1, 8}},     {29, {256, 56}},
                 {30, {1, 2}}};
    for (const auto& e : table)
        if (e.id == type) {
            b = e.s;
            return true;
        }
    return false;
}
constexpr uint32_t T_F32 = 0, T_BF16 = 30, T_IQ3_S = 21;

struct Entry {
    std::string name;
    uint32_t type = 0;
    int n_dims = 0;
    int64_t ne[4] = {1, 1, 1, 1};
    const uint8_t* data = nullptr;
    size_t nbytes = 0;
    int shard = -1;
    uint64_t offset = 0;
};

// a bounds-checked walk over a mapped header
class Walk {
public:
    Walk(const uint8_t* base, size_t size) : base_(base), at_(0), size_(size) {}
    template <typename T>
    T take() {
        if (size_ - at_ < sizeof(T)) throw std::runtime_error("gguf: truncated header");
        T v;
        std::memcpy(&v, base_ + at_, sizeof(T));
        at_ += sizeof(T);
        return v;
    }
    std::string text() {
        const uint64_t n = take<uint64_t>();
        if (n > size_ - at_) throw std::runtime_error("gguf: truncated string");
        std::string s(reinterpret_cast<const char*>(base_ + at_), (size_t) n);
        at_ += (size_t) n;
        return s;
    }
    void skip(uint64_t n) {
        if (n > size_ - at_) throw std::runtime_error("gguf: truncated header");
        at_ += (size_t) n;
    }
    size_t at() const { return at_; }

private:
    const uint8_t* base_;
    size_t at_, size_;
};

// GGUF metadata value types: 0 u8, 1 i8, 2 u16, 3 i16, 4 u32, 5 i32, 6 f32, 7 bool, 8 string, 9 array, 10 u64, 11 i64, 12 f64
inline int scalar_bytes(uint32_t vt) {
    switch (vt) {
        case 0: case 1: case 7: return 1;
        case 2: case 3: return 2;
        case 4: case 5: case 6: return 4;
        case 10: case 11: case 12: return 8;
    }
    return -1;
}
inline bool take_integer(Walk& w, uint32_t vt, int64_t& v) {
    switch (vt) {
        case 0: case 7: v = w.take<uint8_t>(); return true;
        case 1: v = w.take<int8_t>(); return true;
        case 2: v = w.take<uint16_t>(); return true;
        case 3: v = w.take<int16_t>(); return true;
        case 4: v = w.take<uint32_t>(); return true;
        case 5: v = w.take<int32_t>(); return true;
        case 10: v = (int64_t) w.take<uint64_t>(); return true;
        case 11: v = w.take<int64_t>(); return true;
    }
    return false;
}

}  // namespace gguf
}  // namespace fnx

struct fnx_gguf {
    struct Mapping {
        void* base = nullptr;
        size_t size = 0;
        int fd = -1;
        std::string path;
    };
    std::vector<Mapping> maps;
    std::map<std::string, fnx::gguf::Entry> tensors;   // by name
    std::vector<const fnx::gguf::Entry*> order;        // the same, for access by index
    std::map<std::string, int64_t> ints;
    std::map<std::string, double> floats;
    std::map<std::string, std::string> strings;
    std::map<std::string, std::vector<int64_t>> int_arrays;
    std::map<std::string, int> keys;   // every key of the first shard -> its value type

    void unmap() {
        for (Mapping& m : maps) {
            if (m.base && m.base != MAP_FAILED) munmap(m.base, m.size);
            if (m.fd >= 0) close(m.fd);
        }
        maps.clear();
    }
    ~fnx_gguf() { unmap(); }
    fnx_gguf(const fnx_gguf&) = delete;
    fnx_gguf& operator=(const fnx_gguf&) = delete;

    // one file: its metadata (kept for the first shard only) and its tensors
    void add_file(const std::string& path, bool keep_meta) {
        using namespace fnx::gguf;
        Mapping m;
        m.path = path;
        m.fd = open(path.c_str(), O_RDONLY);
        if (m.fd < 0) throw std::runtime_error("gguf: cannot open " + path);
        struct stat sb;
        if (fstat(m.fd, &sb) != 0 || sb.st_size <= 0) {
            close(m.fd);
            throw std::runtime_error("gguf: cannot size " + path);
        }
        m.size = (size_t) sb.st_size;
        m.base = mmap(nullptr, m.size, PROT_READ, MAP_SHARED, m.fd, 0);
        if (m.base == MAP_FAILED) {
            close(m.fd);
            throw std::runtime_error("gguf: mmap failed for " + path);
        }
        maps.push_back(m);
        const int shard = (int) maps.size() - 1;
        const uint8_t* base = static_cast<const uint8_t*>(m.base);
        Walk w(base, m.size);
        if (w.take<uint32_t>() != 0x46554747u) throw std::runtime_error("gguf: bad magic in " + path);
        w.take<uint32_t>();   // version
        const uint64_t n_tensors = w.take<uint64_t>(), n_keys = w.take<uint64_t>();
        uint64_t align = 32;
        for (uint64_t i = 0; i < n_keys; ++i) {
            const std::string key = w.text();
            const uint32_t vt = w.take<uint32_t>();
            if (keep_meta) keys[key] = (int) vt;
            int64_t iv;
            if (vt == 8) {
                std::string v = w.text();
                if (keep_meta) strings[key] = std::move(v);
            } else if (vt == 9) {
                const uint32_t et = w.take<uint32_t>();
                const uint64_t n = w.take<uint64_t>();
                if (et == 8) {
                    for (uint64_t k = 0; k < n; ++k) w.text();
                } else {
                    const int sz = scalar_bytes(et);
                    if (sz < 0) throw std::runtime_error("gguf: nested array in " + key);
                    if (keep_meta && et != 6 && et != 12) {
                        std::vector<int64_t> v;
                        v.reserve((size_t) std::min<uint64_t>(n, 1u << 20));
                        for (uint64_t k = 0; k < n; ++k) {
                            take_integer(w, et, iv);
                            v.push_back(iv);
                        }
                        int_arrays[key] = std::move(v);
                    } else {
                        if (n > (uint64_t) -1 / (uint64_t) sz) throw std::runtime_error("gguf: truncated header");
                        w.skip(n * (uint64_t) sz);
                    }
                }
            } else if (vt == 6) {
                const float v = w.take<float>();
                if (keep_meta) floats[key] = v;
            } else if (vt == 12) {
                const double v = w.take<double>();
                if (keep_meta) floats[key] = v;
            } else if (take_integer(w, vt, iv)) {
                if (keep_meta) ints[key] = iv;
                if (key == "general.alignment") {
                    if (iv < 1) throw std::runtime_error("gguf: general.alignment " + std::to_string(iv) + " in " + path);
                    align = (uint64_t) iv;
                }
            } else {
                throw std::runtime_error("gguf: value type " + std::to_string(vt) + " of " + key + " in " + path);
            }
        }
        std::vector<Entry> found;
        for (uint64_t i = 0; i < n_tensors; ++i) {
            Entry e;
            e.name = w.text();
            const uint32_t nd = w.take<uint32_t>();
            if (nd < 1 || nd > 4)
                throw std::runtime_error("gguf: tensor " + e.name + " has " + std::to_string(nd) + " dimensions in " + path + " (1 to 4 allowed)");
            e.n_dims = (int) nd;
            for (int d = 0; d < e.n_dims; ++d) {
                const uint64_t ne = w.take<uint64_t>();
                if (ne < 1 || ne > (uint64_t) INT64_MAX)
                    throw std::runtime_error("gguf: tensor " + e.name + " has size " + std::to_string(ne) + " in dimension " + std::to_string(d) +
                                             " in " + path);
                e.ne[d] = (int64_t) ne;
            }
            e.type = w.take<uint32_t>();
            e.offset = w.take<uint64_t>();   // relative to the data section until placed below
            e.shard = shard;
            found.push_back(std::move(e));
        }
        const uint64_t data0 = ((uint64_t) w.at() + align - 1) / align * align;
        for (Entry& e : found) {
            BlockShape bs;
            if (!block_shape(e.type, bs)) throw std::runtime_error("gguf: tensor " + e.name + " has unknown ggml type " + std::to_string(e.type) + " in " + path);
            // checked arithmetic throughout: a product that wraps would pass the end test
            uint64_t count = 1, nbytes = 0, end = 0;
            for (int d = 0; d < 4; ++d)
                if (__builtin_mul_overflow(count, (uint64_t) e.ne[d], &count))
                    throw std::runtime_error("gguf: tensor " + e.name + "'s element count overflows in " + path);
            if (__builtin_mul_overflow(count / (uint64_t) bs.values, (uint64_t) bs.bytes, &nbytes) || __builtin_add_overflow(data0, e.offset, &end) ||
                __builtin_add_overflow(end, nbytes, &end) || end > m.size)
                throw std::runtime_error("gguf: tensor " + e.name + " runs past the end of " + path);
            e.nbytes = (size_t) nbytes;
            e.offset += data0;
            e.data = base + e.offset;
            tensors[e.name] = e;
        }
    }

    explicit fnx_gguf(const std::string& first) {
        try {
            add_set(first);
        } catch (...) {
            unmap();   // a constructor that throws runs no destructor
            throw;
        }
        for (const auto& kv : tensors) order.push_back(&kv.second);
    }
    void add_set(const std::string& first) {
        // "<stem>-00001-of-0000M.gguf": every shard of the set, the metadata from the first
        const size_t n = first.size();
        const auto digits = [&](size_t at) {
            for (size_t i = 0; i < 5; ++i)
                if (first[at + i] < '0' || first[at + i] > '9') return false;
            return true;
        };
        // tail: -DDDDD-of-DDDDD.gguf = 1 + 5 + 4 + 5 + 5 = 20 characters
        if (n >= 20 && first.compare(n - 5, 5, ".gguf") == 0 && first.compare(n - 14, 4, "-of-") == 0 && first[n - 20] == '-' && digits(n - 19) &&
            digits(n - 10)) {
            const int total = std::stoi(first.substr(n - 10, 5));
            for (int i = 1; i <= total; ++i) {
                char num[16];
                std::snprintf(num, sizeof num, "%05d", i);
                add_file(first.substr(0, n - 19) + num + first.substr(n - 14), i == 1);
            }
        } else {
            add_file(first, true);
        }
    }
};

namespace fnx {
namespace gguf {

inline void describe(const Entry& e, fnx_gguf_tensor* t) {
    t->name = e.name.c_str();
    t->type = e.type;
    t->n_dims = e.n_dims;
    for (int d = 0; d < 4; ++d) t->ne[d] = e.ne[d];
    t->data = e.data;
    t->nbytes = e.nbytes;
    t->shard = e.shard;
    t->offset = e.offset;
}
inline size_t row_bytes(const fnx_gguf_tensor& t) {
    BlockShape bs;
    if (!block_shape(t.type, bs)) throw std::runtime_error(std::string("gguf: tensor ") + t.name + " has unknown ggml type " + std::to_string(t.type));
    return (size_t) (t.ne[0] / bs.values) * (size_t) bs.bytes;
}
inline std::string nm(const fnx_gguf_tensor& t) { return t.name ? t.name : "(unnamed)"; }
inline void need_rows(const fnx_gguf_tensor& t, int r0, int r1) {
    if (r0 < 0 || r1 <= r0 || r1 > t.ne[1])
        throw std::runtime_error(nm(t) + ": rows [" + std::to_string(r0) + ", " + std::to_string(r1) + ") asked for, it has " + std::to_string(t.ne[1]) +
                                 " a matrix");
}
// per expert: rows [r0, r1) of gate, then of up (model.cpp:722-741). Returns the bytes written (experts * stride).
inline size_t expert_rows2(const fnx_gguf_tensor& g, const fnx_gguf_tensor& u, int r0, int r1, uint8_t* dst, size_t dst_bytes, fnx_dw* w, size_t* stride) {
    if (g.type != u.type || g.ne[0] != u.ne[0] || g.ne[2] != u.ne[2]) throw std::runtime_error(nm(g) + " and " + nm(u) + " do not stack");
    need_rows(g, r0, r1);
    need_rows(u, r0, r1);
    const size_t rb = row_bytes(g), half = (size_t) (r1 - r0) * rb, st = 2 * half, nexp = (size_t) g.ne[2];
    const size_t g_mat = (size_t) g.ne[1] * rb, u_mat = (size_t) u.ne[1] * rb;
    if (w) {
        w->p = dst;
        w->type = g.type;
        w->n_in = (int) g.ne[0];
        w->n_out = 2 * (r1 - r0);
        w->row_bytes = rb;
        w->ep = nullptr;
    }
    if (stride) *stride = st;
    if (!dst) return nexp * st;
    if (dst_bytes < nexp * st) throw std::runtime_error(nm(g) + ": the buffer holds " + std::to_string(dst_bytes) + " bytes, " + std::to_string(nexp * st) + " needed");
    for (size_t e = 0; e < nexp; ++e) {
        std::memcpy(dst + e * st, static_cast<const uint8_t*>(g.data) + e * g_mat + (size_t) r0 * rb, half);
        std::memcpy(dst + e * st + half, static_cast<const uint8_t*>(u.data) + e * u_mat + (size_t) r0 * rb, half);
    }
    return nexp * st;
}
// per expert: every row, columns [c0, c1) (model.cpp:768-790, which counts in 32-value blocks; here the columns must be
// whole blocks of the tensor's own type, 256 for IQ3_S)
inline size_t expert_cols(const fnx_gguf_tensor& t, int c0, int c1, uint8_t* dst, size_t dst_bytes, fnx_dw* w, size_t* stride) {
    BlockShape bs;
    if (!block_shape(t.type, bs)) throw std::runtime_error(nm(t) + ": unknown ggml type " + std::to_string(t.type));
    if (c0 < 0 || c1 <= c0 || c1 > t.ne[0] || c0 % bs.values || c1 % bs.values)
        throw std::runtime_error(nm(t) + ": columns [" + std::to_string(c0) + ", " + std::to_string(c1) + ") asked for, a row has " + std::to_string(t.ne[0]) +
                                 " in blocks of " + std::to_string(bs.values));
    const size_t src_row = row_bytes(t), rb = (size_t) (c1 - c0) / bs.values * bs.bytes, at = (size_t) c0 / bs.values * bs.bytes;
    const size_t rows = (size_t) t.ne[1], nexp = (size_t) t.ne[2], st = rows * rb, src_mat = rows * src_row;
    if (w) {
        w->p = dst;
        w->type = t.type;
        w->n_in = c1 - c0;
        w->n_out = (int) rows;
        w->row_bytes = rb;
        w->ep = nullptr;
    }
    if (stride) *stride = st;
    if (!dst) return nexp * st;
    if (dst_bytes < nexp * st) throw std::runtime_error(nm(t) + ": the buffer holds " + std::to_string(dst_bytes) + " bytes, " + std::to_string(nexp * st) + " needed");
    for (size_t e = 0; e < nexp; ++e)
        for (size_t r = 0; r < rows; ++r)
            std::memcpy(dst + e * st + r * rb, static_cast<const uint8_t*>(t.data) + e * src_mat + r * src_row + at, rb);
    return nexp * st;
}
// the router's rows, then the shared expert's gate row, as f32 (model.cpp:988-989; F32 or BF16 in the file)
inline void router_rows(const fnx_gguf_tensor& gi, const fnx_gguf_tensor& gs, float* dst) {
    if (gi.ne[0] != gs.ne[0]) throw std::runtime_error(nm(gi) + " and " + nm(gs) + " do not stack");
    size_t at = 0;
    for (const fnx_gguf_tensor* t : {&gi, &gs}) {
        const size_t n = (size_t) (t->ne[0] * t->ne[1]);
        if (t->type == T_F32) std::memcpy(dst + at, t->data, n * 4);
        else if (t->type == T_BF16)
            for (size_t i = 0; i < n; ++i) {
                const uint32_t bits = (uint32_t) static_cast<const uint16_t*>(t->data)[i] << 16;
                std::memcpy(dst + at + i, &bits, 4);
            }
        else throw std::runtime_error(nm(*t) + ": router rows must be F32 or BF16, not ggml type " + std::to_string(t->type));
        at += n;
    }
}

}  // namespace gguf
}  // namespace fnx
