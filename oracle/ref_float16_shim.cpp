// Thin extern "C" view of the reference's own float16 class, compiled together with the
// reference's src/vpux_utils/src/core/type/float16.cpp (taken from the reference checkout at
// build time, never copied).  TEST INFRASTRUCTURE ONLY: used to validate oracle/vpx_oracle.c.
#include <vpux/utils/core/type/float16.hpp>

#include <cstddef>
#include <cstdint>

extern "C" {
uint16_t ref_f32_to_f16(float v) {
    return vpux::type::float16(v).to_bits();
}
float ref_f16_to_f32(uint16_t bits) {
    return static_cast<float>(vpux::type::float16::from_bits(bits));
}
// float16::operator+ (fp32 add, then round), float16.hpp:123-126
uint16_t ref_f16_add(uint16_t a, uint16_t b) {
    return (vpux::type::float16::from_bits(a) + vpux::type::float16::from_bits(b)).to_bits();
}
void ref_f32_to_f16_array(const float* in, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = vpux::type::float16(in[i]).to_bits();
}
void ref_f16_to_f32_array(const uint16_t* in, float* out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = static_cast<float>(vpux::type::float16::from_bits(in[i]));
}
void ref_f16_add_array(const uint16_t* a, const uint16_t* b, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; i++)
        out[i] = (vpux::type::float16::from_bits(a[i]) + vpux::type::float16::from_bits(b[i])).to_bits();
}
}
