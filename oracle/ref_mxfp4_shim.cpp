// C entry points around the reference's own MXFP4 codec header, compiled from
// the reference tree where it lies (it needs nothing but the standard library).
// TEST INFRASTRUCTURE: used only to validate oracle/moe_oracle.c.
// Wraps include/coalsack/gguf/gguf_dequant.h:419-455 of the reference.
#include <cstdint>

#include "coalsack/gguf/gguf_dequant.h"

extern "C" {
float ref_e8m0_to_fp32_half(uint8_t x) { return coalsack::e8m0_to_fp32_half(x); }
void ref_dequantize_block_mxfp4(const uint8_t* src, float* dst, int64_t k) {
  coalsack::dequantize_block_mxfp4(src, dst, k);
}
}
