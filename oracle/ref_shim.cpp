// TEST INFRASTRUCTURE. C entry points around the reference's own CPU block code, so tests can call it through ctypes.
// Compiled together with the reference's engine/core/gguf_quant.cpp, gguf.cpp and gguf_convert.cpp where they lie
// (see the Makefile); nothing of the reference is copied here. Only the declarations of core/gguf_quant.hpp are used.
#include <cstdint>

#include "core/gguf_quant.hpp"

extern "C" {

// yah::core::QuantizeQ8_0 (engine/core/gguf_quant.cpp:310-320)
void ref_quantize_q8_0(const float* x, std::uint64_t n, std::uint8_t* dst) { yah::core::QuantizeQ8_0(x, n, dst); }

// yah::core::Dequantize for Q8_0 / Q4_0 (engine/core/gguf_quant.cpp:72-75, 48-51, 290-308)
void ref_dequantize_q8_0(const std::uint8_t* src, std::uint64_t n, float* dst) {
  yah::core::Dequantize(yah::core::GgmlType::kQ8_0, src, dst, n);
}
void ref_dequantize_q4_0(const std::uint8_t* src, std::uint64_t n, float* dst) {
  yah::core::Dequantize(yah::core::GgmlType::kQ4_0, src, dst, n);
}
// f16 / bf16 arrays to f32 through the same function (gguf_quant.cpp:293-300)
void ref_f16_to_f32(const std::uint8_t* src, std::uint64_t n, float* dst) {
  yah::core::Dequantize(yah::core::GgmlType::kF16, src, dst, n);
}
void ref_bf16_to_f32(const std::uint8_t* src, std::uint64_t n, float* dst) {
  yah::core::Dequantize(yah::core::GgmlType::kBF16, src, dst, n);
}
}
