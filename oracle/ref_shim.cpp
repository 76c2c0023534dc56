// Thin C wrapper around the OpenVINO reference's own sub-byte iterator and float16
// class, compiled from the reference tree where it lies (see Makefile, target _ref).
// TEST INFRASTRUCTURE ONLY: used to check oracle.c, never loaded by the product.
//
// Wraps: src/core/dev_api/openvino/core/type/element_iterator.hpp (ov::element::iterator<ET>)
//        src/core/src/type/float16.cpp (ov::float16)
#include <cstddef>
#include <cstdint>

#include "openvino/core/type/element_iterator.hpp"
#include "openvino/core/type/float16.hpp"

extern "C" {

void ref_unpack_u4(const uint8_t* src, size_t n, uint8_t* dst) {
    auto it = ov::element::iterator<ov::element::u4>(reinterpret_cast<const int8_t*>(src));
    for (size_t i = 0; i < n; ++i, ++it)
        dst[i] = static_cast<uint8_t>(static_cast<int8_t>(*it));
}

void ref_unpack_i4(const uint8_t* src, size_t n, int8_t* dst) {
    auto it = ov::element::iterator<ov::element::i4>(reinterpret_cast<const int8_t*>(src));
    for (size_t i = 0; i < n; ++i, ++it)
        dst[i] = static_cast<int8_t>(*it);
}

void ref_pack_u4(const uint8_t* src, size_t n, uint8_t* dst) {
    auto it = ov::element::iterator<ov::element::u4>(reinterpret_cast<int8_t*>(dst));
    for (size_t i = 0; i < n; ++i, ++it)
        *it = static_cast<int8_t>(src[i]);
}

void ref_pack_i4(const int8_t* src, size_t n, uint8_t* dst) {
    auto it = ov::element::iterator<ov::element::i4>(reinterpret_cast<int8_t*>(dst));
    for (size_t i = 0; i < n; ++i, ++it)
        *it = src[i];
}

uint16_t ref_f32_to_f16(float f) {
    return ov::float16(f).to_bits();
}

float ref_f16_to_f32(uint16_t h) {
    return static_cast<float>(ov::float16::from_bits(h));
}

}  // extern "C"
