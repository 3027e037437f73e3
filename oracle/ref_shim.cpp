// Thin C wrapper around the reference's own host-only conversion header, compiled from where it lies
// (engine/src/tensor_convert.hpp under the reference root, passed with -I). Used by the tests to pin the oracle's
// half conversions, codebook and IQ3_S decoder against the reference's code itself. TEST INFRASTRUCTURE ONLY; the
// built library goes to oracle/_ref/ and is never committed.
#include <cstddef>
#include <cstdint>

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
}
