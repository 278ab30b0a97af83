/* quant.c — block codecs (see quant.h).  Dequantization restates the reference's
 * src/quant.c:269-343 for the supported types; values are identical because each
 * is a single f32 multiply of an exactly converted scale and a small integer. */
#include <stdlib.h>
#include <string.h>
#include <math.h>

#include "quant.h"
#include "../../include/lg_math.h"

struct traits { uint32_t id; const char *name; int blck; size_t bytes; };
static const struct traits k_traits[] = {
    { GGML_TYPE_F32, "f32", 1, 4 },   { GGML_TYPE_F16, "f16", 1, 2 },  { GGML_TYPE_BF16, "bf16", 1, 2 },
    { GGML_TYPE_Q4_0, "q4_0", 32, LG_Q4_0_BYTES }, { GGML_TYPE_Q8_0, "q8_0", 32, 34 },
    /* named but not decoded */
    { GGML_TYPE_Q2_K, "q2_K", 0, 0 }, { GGML_TYPE_Q3_K, "q3_K", 0, 0 }, { GGML_TYPE_Q4_K, "q4_K", 0, 0 },
    { GGML_TYPE_Q5_K, "q5_K", 0, 0 }, { GGML_TYPE_Q6_K, "q6_K", 0, 0 },
};
static const struct traits *find(uint32_t type) {
    for (size_t i = 0; i < sizeof k_traits / sizeof k_traits[0]; i++)
        if (k_traits[i].id == type) return &k_traits[i];
    return NULL;
}

const char *ggml_type_name(uint32_t type) { const struct traits *t = find(type); return t ? t->name : "?"; }
int    ggml_blck_size(uint32_t type) { const struct traits *t = find(type); return t ? t->blck : 0; }
size_t ggml_type_size(uint32_t type) { const struct traits *t = find(type); return t ? t->bytes : 0; }

size_t ggml_nbytes(uint32_t type, int64_t n) {
    const struct traits *t = find(type);
    if (!t || !t->blck || n < 0 || n % t->blck) return 0;
    return (size_t)(n / t->blck) * t->bytes;
}

bool dequantize_into(uint32_t type, const void *src, float *out, int64_t n) {
    const struct traits *t = find(type);
    if (!t || !t->blck || n % t->blck) return false;
    const unsigned char *p = src;
    switch (type) {
    case GGML_TYPE_F32:
        memcpy(out, src, (size_t)n * 4);
        return true;
    case GGML_TYPE_F16:
        for (int64_t i = 0; i < n; i++) { uint16_t h; memcpy(&h, p + 2 * i, 2); out[i] = lg_f16_to_f32(h); }
        return true;
    case GGML_TYPE_BF16:
        for (int64_t i = 0; i < n; i++) { uint16_t h; memcpy(&h, p + 2 * i, 2); out[i] = lg_bits_to_f32((uint32_t)h << 16); }
        return true;
    case GGML_TYPE_Q4_0:
        for (int64_t b = 0; b < n / 32; b++, p += LG_Q4_0_BYTES, out += 32) {
            uint16_t h; memcpy(&h, p, 2);
            const float d = lg_f16_to_f32(h);
            for (int j = 0; j < 16; j++) {
                out[j]      = d * (float)((int)(p[2 + j] & 15) - 8);
                out[j + 16] = d * (float)((int)(p[2 + j] >> 4) - 8);
            }
        }
        return true;
    case GGML_TYPE_Q8_0:
        for (int64_t b = 0; b < n / 32; b++, p += 34, out += 32) {
            uint16_t h; memcpy(&h, p, 2);
            const float d = lg_f16_to_f32(h);
            for (int j = 0; j < 32; j++) out[j] = d * (float)(int8_t)p[2 + j];
        }
        return true;
    default:
        return false;
    }
}

float *dequantize_row(const struct gguf_tensor *t, int64_t row, int64_t row_len) {
    int blck = ggml_blck_size(t->type);
    if (!t->data || !blck || row_len % blck || (row * row_len) % blck) return NULL;
    const unsigned char *src = (const unsigned char *)t->data + (size_t)(row * row_len / blck) * ggml_type_size(t->type);
    float *y = malloc((size_t)row_len * sizeof(float));
    if (y && !dequantize_into(t->type, src, y, row_len)) { free(y); y = NULL; }
    return y;
}

float *dequantize(const struct gguf_tensor *t) {
    int64_t n = 1;
    for (uint32_t i = 0; i < t->n_dims; i++) n *= (int64_t)t->dims[i];
    return dequantize_row(t, 0, n);
}

void lg_quantize_q4_0(const float *x, void *out, int64_t n) {
    unsigned char *p = out;
    for (int64_t b = 0; b < n / 32; b++, x += 32, p += LG_Q4_0_BYTES) {
        float amax = 0.0f, mx = 0.0f;
        for (int j = 0; j < 32; j++) if (fabsf(x[j]) > amax) { amax = fabsf(x[j]); mx = x[j]; }
        const float d = mx / -8.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
        uint16_t h = lg_f32_to_f16(d);
        memcpy(p, &h, 2);
        for (int j = 0; j < 16; j++) {
            int lo = (int)(x[j] * id + 8.5f), hi = (int)(x[j + 16] * id + 8.5f);
            if (lo > 15) lo = 15;
            if (hi > 15) hi = 15;
            p[2 + j] = (unsigned char)(lo | (hi << 4));
        }
    }
}
