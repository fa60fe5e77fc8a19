// C entry points around the reference's own MXFP4 codec header, compiled from
// the reference tree where it lies (it needs nothing but the standard library).
// TEST INFRASTRUCTURE: used only to validate oracle/moe_oracle.c.
// Wraps include/coalsack/gguf/gguf_dequant.h:419-455 of the reference, and its
// K-quant codecs and fp32 -> fp16 conversion (:149-258, :458-487) composed the way
// src/llm/moe_weight_provider.cpp:17-33 widens Q4_K / Q6_K experts to fp16.
#include <vector>
#include <cstdint>

#include "coalsack/gguf/gguf_dequant.h"

extern "C" {
float ref_e8m0_to_fp32_half(uint8_t x) { return coalsack::e8m0_to_fp32_half(x); }
void ref_dequantize_block_mxfp4(const uint8_t* src, float* dst, int64_t k) {
  coalsack::dequantize_block_mxfp4(src, dst, k);
}
void ref_dequantize_block_q4_K(const uint8_t* src, float* dst, int64_t k) {
  coalsack::dequantize_block_q4_K(src, dst, k);
}
void ref_dequantize_block_q6_K(const uint8_t* src, float* dst, int64_t k) {
  coalsack::dequantize_block_q6_K(src, dst, k);
}
uint16_t ref_fp32_to_fp16(float f) { return coalsack::fp32_to_fp16(f); }
float ref_fp16_to_fp32(uint16_t h) { return coalsack::fp16_to_fp32(h); }
void ref_q4k_to_fp16(const uint8_t* src, uint16_t* dst, int64_t k) {
  std::vector<float> temp((size_t)k);
  coalsack::dequantize_block_q4_K(src, temp.data(), k);
  for (int64_t i = 0; i < k; ++i) dst[i] = coalsack::fp32_to_fp16(temp[(size_t)i]);
}
void ref_q6k_to_fp16(const uint8_t* src, uint16_t* dst, int64_t k) {
  std::vector<float> temp((size_t)k);
  coalsack::dequantize_block_q6_K(src, temp.data(), k);
  for (int64_t i = 0; i < k; ++i) dst[i] = coalsack::fp32_to_fp16(temp[(size_t)i]);
}
}
