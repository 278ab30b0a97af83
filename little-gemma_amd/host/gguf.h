/* gguf.h — GGUF v2/v3 container: reader with the reference's public shape, plus a writer.
 *
 * Struct layouts, enum values and reader entry points match the reference's
 * include/gguf.h:8-136 so a backend translation unit written against this
 * header also compiles against the reference's own (the link-time seam,
 * CMakeLists.txt:42-45).  The lg_gw_* writer has no reference counterpart: the
 * reference only reads GGUF; the writer exists to produce the seeded synthetic
 * models the parity tests and the benchmark run on.
 */
#ifndef GGUF_H
#define GGUF_H

#include <stdint.h>
#include <stdbool.h>
#include <stdio.h>
#include <stddef.h>

#define GGUF_MAGIC_LE 0x46554747u   /* "GGUF" read little-endian */
#define GGUF_MAGIC_BE 0x47475546u   /* same bytes on a big-endian file: rejected */

enum gguf_type {
    GGUF_TYPE_UINT8 = 0, GGUF_TYPE_INT8 = 1, GGUF_TYPE_UINT16 = 2, GGUF_TYPE_INT16 = 3,
    GGUF_TYPE_UINT32 = 4, GGUF_TYPE_INT32 = 5, GGUF_TYPE_FLOAT32 = 6, GGUF_TYPE_BOOL = 7,
    GGUF_TYPE_STRING = 8, GGUF_TYPE_ARRAY = 9, GGUF_TYPE_UINT64 = 10, GGUF_TYPE_INT64 = 11,
    GGUF_TYPE_FLOAT64 = 12, GGUF_TYPE_COUNT,
};

struct gguf_header {
    uint32_t magic;
    uint32_t version;
    uint64_t num_tensors;
    uint64_t num_meta;
};

struct gguf_meta {
    char    *key;
    uint32_t type;
    union {
        uint8_t u8; int8_t i8; uint16_t u16; int16_t i16;
        uint32_t u32; int32_t i32; uint64_t u64; int64_t i64;
        float f32; double f64; bool bool_;
        char *str;
        struct { uint32_t type; uint64_t n; void *data; } arr;   /* strings: char*[n] */
    } value;
};

struct gguf_tensor {
    char    *name;
    uint32_t n_dims;
    uint64_t dims[4];     /* dims[0] = row length (contraction axis), dims[1] = rows */
    uint32_t type;        /* ggml type id */
    uint64_t offset;      /* from the start of the data section */
    void    *data;
};

struct gguf_context {
    struct gguf_header  header;
    struct gguf_meta   *meta;
    struct gguf_tensor *tensors;
    size_t              alignment;
    size_t              data_offset;
    void   *data;
    size_t  data_size;
    void   *map_base;
    size_t  map_len;
    int     map_fd;
};

size_t      gguf_type_size(uint32_t type);
const char *gguf_type_name(uint32_t type);

struct gguf_context *load_gguf(const char *filepath);
void free_gguf(struct gguf_context *ctx);
void gguf_data_dontneed(const struct gguf_context *ctx, const void *p, size_t bytes);
void gguf_set_max_data_bytes(size_t max_bytes);
void gguf_dump(const struct gguf_context *ctx);

const struct gguf_meta   *gguf_find_meta(const struct gguf_context *ctx, const char *key);
const struct gguf_tensor *gguf_find_tensor(const struct gguf_context *ctx, const char *name);
uint32_t    gguf_get_u32(const struct gguf_context *ctx, const char *key, uint32_t fallback);
int32_t     gguf_get_i32(const struct gguf_context *ctx, const char *key, int32_t fallback);
float       gguf_get_f32(const struct gguf_context *ctx, const char *key, float fallback);
const char *gguf_get_str(const struct gguf_context *ctx, const char *key, const char *fallback);

/* ---- writer ------------------------------------------------------------- */
/* Declare metadata and tensors, then lg_gw_commit() sizes the file, maps it and
 * returns; lg_gw_tensor_data() gives each tensor's bytes to fill in place;
 * lg_gw_close() flushes.  All functions return 0 / non-NULL on success. */
struct lg_gguf_writer;
struct lg_gguf_writer *lg_gw_open(const char *path, uint32_t version, uint32_t alignment);
int lg_gw_meta_u32(struct lg_gguf_writer *w, const char *key, uint32_t v);
int lg_gw_meta_f32(struct lg_gguf_writer *w, const char *key, float v);
int lg_gw_meta_str(struct lg_gguf_writer *w, const char *key, const char *v);
int lg_gw_meta_array(struct lg_gguf_writer *w, const char *key, uint32_t elem_type,
                     uint64_t n, const void *data);
int lg_gw_meta_empty_strings(struct lg_gguf_writer *w, const char *key, uint64_t n);
int lg_gw_add_tensor(struct lg_gguf_writer *w, const char *name, uint32_t ggml_type,
                     uint32_t n_dims, const uint64_t *dims);      /* returns tensor index or -1 */
int lg_gw_commit(struct lg_gguf_writer *w);
void *lg_gw_tensor_data(struct lg_gguf_writer *w, int index, size_t *bytes);
int lg_gw_close(struct lg_gguf_writer *w);

#endif /* GGUF_H */
