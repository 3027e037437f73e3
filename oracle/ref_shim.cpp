// Thin C wrapper around the reference's own host-only conversion header and GGUF reader, compiled from where they lie
// (engine/src/tensor_convert.hpp, gguf.hpp and gguf.cpp under the reference root, passed with -I and on the compile
// line). Used by the tests to pin the oracle's half conversions, codebook and IQ3_S decoder, and the library's GGUF
// header walk, against the reference's code itself. TEST INFRASTRUCTURE ONLY; the built library goes to oracle/_ref/
// and is never committed.
#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <stdexcept>
#include <string>

#include "gguf.hpp"
#include "tensor_convert.hpp"

extern "C" {
float fnx_ref_h2f(uint16_t h) { return fnx::conv::h2f(h); }
uint16_t fnx_ref_f2h(float x) { return fnx::conv::f2h(x); }
const uint32_t* fnx_ref_iq3s_grid() { return fnx::conv::iq3s_grid(); }
// type 21 = IQ3_S, 8 = Q8_0 (gguf.hpp:22-27)
int fnx_ref_dequantize(uint32_t type, const uint8_t* src, size_t n, float* y) {
    try {
        fnx::conv::dequantize(type, src, n, y);
        return 0;
    } catch (...) {
        return 1;
    }
}
void fnx_ref_quantize_q8_0(const float* x, size_t n, uint8_t* dst) { fnx::conv::quantize_q8_0(x, n, dst); }

// the reference's GGUF reader (gguf.hpp:25-45): open (null and a message when it refuses the file), tensors in name
// order, metadata
void* fnx_ref_gguf_open(const char* path, char* err, size_t err_cap) {
    try {
        return new fnx::Gguf(path);
    } catch (const std::exception& e) {
        if (err && err_cap) std::snprintf(err, err_cap, "%s", e.what());
        return nullptr;
    }
}
void fnx_ref_gguf_close(void* g) { delete static_cast<fnx::Gguf*>(g); }
int fnx_ref_gguf_count(void* g) { return (int) static_cast<fnx::Gguf*>(g)->tensors().size(); }
int fnx_ref_gguf_shards(void* g) { return static_cast<fnx::Gguf*>(g)->shards(); }
// the i-th tensor in name order; info = {type, n_dims, ne0..ne3, nbytes, shard, offset, row_bytes}
int fnx_ref_gguf_tensor(void* g, int i, char* name, size_t name_cap, int64_t* info) {
    const auto& ts = static_cast<fnx::Gguf*>(g)->tensors();
    if (i < 0 || i >= (int) ts.size()) return 1;
    auto it = ts.begin();
    std::advance(it, i);
    const fnx::Tensor& t = it->second;
    std::snprintf(name, name_cap, "%s", t.name.c_str());
    info[0] = t.type;
    info[1] = t.n_dims;
    for (int d = 0; d < 4; ++d) info[2 + d] = t.ne[d];
    info[6] = (int64_t) t.nbytes;
    info[7] = t.shard;
    info[8] = (int64_t) t.offset;
    info[9] = (int64_t) t.row_bytes();
    return 0;
}
const void* fnx_ref_gguf_data(void* g, const char* name) {
    const fnx::Tensor* t = static_cast<fnx::Gguf*>(g)->find(name);
    return t ? t->data : nullptr;
}
int fnx_ref_gguf_has_key(void* g, const char* key) { return static_cast<fnx::Gguf*>(g)->has_key(key) ? 1 : 0; }
int fnx_ref_gguf_num(void* g, const char* key, double* v) {
    try {
        *v = static_cast<fnx::Gguf*>(g)->num(key);
        return 0;
    } catch (...) {
        return 1;
    }
}
int fnx_ref_gguf_str(void* g, const char* key, char* out, size_t cap) {
    try {
        std::snprintf(out, cap, "%s", static_cast<fnx::Gguf*>(g)->s(key).c_str());
        return 0;
    } catch (...) {
        return 1;
    }
}
}
