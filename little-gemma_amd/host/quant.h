/* quant.h — ggml block formats the verify path touches.
 *
 * Entry points and type ids follow the reference's include/quant.h:13-51.  Only
 * the formats the synthetic models use are implemented (f32, f16, bf16, q4_0,
 * q8_0); the K-quant ids are listed so an unsupported file is named in the
 * error rather than misread.  lg_quantize_q4_0 has no reference counterpart
 * (the reference only dequantizes): it packs the generator's weights.
 */
#ifndef QUANT_H
#define QUANT_H

#include <stdint.h>
#include <stddef.h>
#include <stdbool.h>

#include "gguf.h"

enum ggml_type {
    GGML_TYPE_F32 = 0, GGML_TYPE_F16 = 1, GGML_TYPE_Q4_0 = 2, GGML_TYPE_Q8_0 = 8,
    GGML_TYPE_Q2_K = 10, GGML_TYPE_Q3_K = 11, GGML_TYPE_Q4_K = 12, GGML_TYPE_Q5_K = 13,
    GGML_TYPE_Q6_K = 14, GGML_TYPE_BF16 = 30,
};

/* 18-byte q4_0 block: f16 scale, then 16 bytes; byte j carries element j in its
 * low nibble and element j+16 in its high nibble; value = d * (nibble - 8). */
#define LG_Q4_0_BLOCK 32
#define LG_Q4_0_BYTES 18

const char *ggml_type_name(uint32_t type);
int         ggml_blck_size(uint32_t type);
size_t      ggml_type_size(uint32_t type);
size_t      ggml_nbytes(uint32_t type, int64_t n_elements);

float *dequantize(const struct gguf_tensor *t);
float *dequantize_row(const struct gguf_tensor *t, int64_t row, int64_t row_len);
bool   dequantize_into(uint32_t type, const void *src, float *out, int64_t n);

/* Pack n (multiple of 32) floats into q4_0 blocks: d = (signed value of largest
 * magnitude) / -8, q = min(15, trunc(x/d + 8.5)). */
void lg_quantize_q4_0(const float *x, void *out, int64_t n);

#endif
