/* gguf.c — GGUF v2/v3 reader (same observable behaviour as the reference's
 * src/gguf.c:249-386,555-599) and the writer used for synthetic models.
 *
 * The reader maps the whole file once and walks the header with a bounds-checked
 * cursor; the tensor-data section is then the tail of that same private mapping.
 * Refusals follow the reference: wrong magic / big-endian / version not in {2,3}
 * (src/gguf.c:263-279), nested arrays (:183), lengths over 1 GiB (:131), tensor
 * offsets past the data section (:369-375), data larger than available memory or
 * the configured cap (:73-88).
 */
#define _GNU_SOURCE
#include <stdlib.h>
#include <string.h>
#include <errno.h>
#include <unistd.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>

#include "gguf.h"
#include "quant.h"

#define LG_GGUF_MAX_LEN (1ull << 30)

static const struct { size_t size; const char *name; } k_types[GGUF_TYPE_COUNT] = {
    {1, "u8"}, {1, "i8"}, {2, "u16"}, {2, "i16"}, {4, "u32"}, {4, "i32"}, {4, "f32"},
    {1, "bool"}, {0, "str"}, {0, "arr"}, {8, "u64"}, {8, "i64"}, {8, "f64"},
};

size_t gguf_type_size(uint32_t type) { return type < GGUF_TYPE_COUNT ? k_types[type].size : 0; }
const char *gguf_type_name(uint32_t type) { return type < GGUF_TYPE_COUNT ? k_types[type].name : "?"; }

static size_t g_data_cap = 0;
void gguf_set_max_data_bytes(size_t max_bytes) { g_data_cap = max_bytes; }

static size_t mem_available(void) {
    FILE *f = fopen("/proc/meminfo", "r");
    if (!f) return 0;
    char line[160];
    unsigned long long kb = 0;
    size_t out = 0;
    while (fgets(line, sizeof line, f))
        if (sscanf(line, "MemAvailable: %llu kB", &kb) == 1) { out = (size_t)kb << 10; break; }
    fclose(f);
    return out;
}

/* ---- cursor over the mapped file ---------------------------------------- */
struct cur { const unsigned char *p, *end; };

static bool take(struct cur *c, void *dst, size_t n) {
    if ((size_t)(c->end - c->p) < n) return false;
    memcpy(dst, c->p, n);
    c->p += n;
    return true;
}

static char *take_string(struct cur *c) {
    uint64_t len;
    if (!take(c, &len, 8) || len > LG_GGUF_MAX_LEN || (uint64_t)(c->end - c->p) < len) return NULL;
    char *s = malloc(len + 1);
    if (!s) return NULL;
    memcpy(s, c->p, len);
    s[len] = 0;
    c->p += len;
    return s;
}

static void meta_release(struct gguf_meta *m) {
    free(m->key);
    if (m->type == GGUF_TYPE_STRING) free(m->value.str);
    else if (m->type == GGUF_TYPE_ARRAY) {
        if (m->value.arr.type == GGUF_TYPE_STRING && m->value.arr.data) {
            char **it = m->value.arr.data;
            for (uint64_t i = 0; i < m->value.arr.n; i++) free(it[i]);
        }
        free(m->value.arr.data);
    }
}

static bool take_meta(struct cur *c, struct gguf_meta *m) {
    if (!(m->key = take_string(c)) || !take(c, &m->type, 4)) return false;
    if (m->type == GGUF_TYPE_STRING) return (m->value.str = take_string(c)) != NULL;
    if (m->type != GGUF_TYPE_ARRAY) {
        size_t sz = gguf_type_size(m->type);
        return sz && take(c, &m->value, sz);
    }
    uint32_t et; uint64_t n;
    if (!take(c, &et, 4) || !take(c, &n, 8) || et == GGUF_TYPE_ARRAY) return false;
    m->value.arr.type = et; m->value.arr.n = n; m->value.arr.data = NULL;
    if (!n) return true;
    if (et == GGUF_TYPE_STRING) {
        if (n > LG_GGUF_MAX_LEN / sizeof(char *)) return false;
        char **it = calloc(n, sizeof(char *));
        if (!it) return false;
        m->value.arr.data = it;
        for (uint64_t i = 0; i < n; i++) if (!(it[i] = take_string(c))) return false;
        return true;
    }
    size_t es = gguf_type_size(et);
    if (!es || n > LG_GGUF_MAX_LEN / es) return false;
    if (!(m->value.arr.data = malloc(n * es))) return false;
    return take(c, m->value.arr.data, n * es);
}

struct gguf_context *load_gguf(const char *filepath) {
    int fd = open(filepath, O_RDONLY);
    if (fd < 0) { perror("Failed to open file"); return NULL; }
    struct stat st;
    struct gguf_context *ctx = NULL;
    void *map = MAP_FAILED;
    if (fstat(fd, &st) != 0 || st.st_size < (off_t)sizeof(struct gguf_header)) {
        fprintf(stderr, "Failed to read header.\n");
        goto fail;
    }
    size_t fsize = (size_t)st.st_size;
    /* private + writable like the reference (src/gguf.c:337-344): a stray store
     * copies a page instead of touching the file */
    map = mmap(NULL, fsize, PROT_READ | PROT_WRITE, MAP_PRIVATE, fd, 0);
    if (map == MAP_FAILED) { perror("mmap"); goto fail; }

    ctx = calloc(1, sizeof *ctx);
    if (!ctx) goto fail;
    ctx->map_fd = -1;
    struct cur c = { map, (const unsigned char *)map + fsize };
    take(&c, &ctx->header, sizeof ctx->header);
    if (ctx->header.magic == GGUF_MAGIC_BE) {
        fprintf(stderr, "Big-endian GGUF files are not supported (this reader assumes little-endian).\n");
        goto fail;
    }
    if (ctx->header.magic != GGUF_MAGIC_LE) { fprintf(stderr, "Invalid GGUF magic number.\n"); goto fail; }
    if (ctx->header.version != 2 && ctx->header.version != 3) {
        fprintf(stderr, "Unsupported GGUF version %u (only 2 and 3 are handled).\n", ctx->header.version);
        goto fail;
    }
    /* counts come off disk: an entry needs at least 12 bytes, so anything larger
     * than the file cannot be honest */
    if (ctx->header.num_meta > fsize / 12 || ctx->header.num_tensors > fsize / 12) {
        fprintf(stderr, "Implausible GGUF entry counts.\n");
        goto fail;
    }
    if (ctx->header.num_meta && !(ctx->meta = calloc(ctx->header.num_meta, sizeof *ctx->meta))) goto fail;
    for (uint64_t i = 0; i < ctx->header.num_meta; i++)
        if (!take_meta(&c, &ctx->meta[i])) {
            fprintf(stderr, "Failed to read KV pair %llu.\n", (unsigned long long)i);
            goto fail;
        }
    if (ctx->header.num_tensors && !(ctx->tensors = calloc(ctx->header.num_tensors, sizeof *ctx->tensors))) goto fail;
    for (uint64_t i = 0; i < ctx->header.num_tensors; i++) {
        struct gguf_tensor *t = &ctx->tensors[i];
        if (!(t->name = take_string(&c)) || !take(&c, &t->n_dims, 4) || t->n_dims < 1 || t->n_dims > 4 ||
            !take(&c, t->dims, 8 * t->n_dims) || !take(&c, &t->type, 4) || !take(&c, &t->offset, 8)) {
            fprintf(stderr, "Failed to read tensor info %llu.\n", (unsigned long long)i);
            goto fail;
        }
    }
    ctx->alignment = 32;
    const struct gguf_meta *al = gguf_find_meta(ctx, "general.alignment");
    if (al && al->type == GGUF_TYPE_UINT32 && al->value.u32) ctx->alignment = al->value.u32;

    size_t used = (size_t)(c.p - (const unsigned char *)map);
    ctx->data_offset = (used + ctx->alignment - 1) / ctx->alignment * ctx->alignment;
    if (ctx->data_offset > fsize) {
        if (ctx->header.num_tensors) { fprintf(stderr, "Invalid file size relative to data offset.\n"); goto fail; }
        ctx->data_offset = fsize;
    }
    ctx->data_size = fsize - ctx->data_offset;
    if (g_data_cap && ctx->data_size > g_data_cap) {
        fprintf(stderr, "Tensor data (%zu bytes) exceeds the configured limit (%zu bytes).\n", ctx->data_size, g_data_cap);
        goto fail;
    }
    size_t avail = mem_available();
    if (avail && ctx->data_size > avail) {
        fprintf(stderr, "Tensor data (%zu bytes) exceeds available memory (%zu bytes); "
                        "refusing to load to avoid paging to disk.\n", ctx->data_size, avail);
        goto fail;
    }
    ctx->map_base = map;
    ctx->map_len = fsize;
    ctx->map_fd = fd;
    ctx->data = ctx->data_size ? (unsigned char *)map + ctx->data_offset : NULL;
    for (uint64_t i = 0; i < ctx->header.num_tensors; i++) {
        struct gguf_tensor *t = &ctx->tensors[i];
        if (t->offset > ctx->data_size) {
            fprintf(stderr, "Tensor '%s' offset out of bounds.\n", t->name);
            ctx->map_base = NULL; ctx->map_fd = -1;
            goto fail;
        }
        t->data = ctx->data ? (unsigned char *)ctx->data + t->offset : NULL;
    }
    return ctx;

fail:
    if (map != MAP_FAILED) munmap(map, (size_t)st.st_size);
    close(fd);
    free_gguf(ctx);
    return NULL;
}

void free_gguf(struct gguf_context *ctx) {
    if (!ctx) return;
    if (ctx->map_base) munmap(ctx->map_base, ctx->map_len);
    if (ctx->map_fd >= 0) close(ctx->map_fd);
    if (ctx->meta) {
        for (uint64_t i = 0; i < ctx->header.num_meta; i++) meta_release(&ctx->meta[i]);
        free(ctx->meta);
    }
    if (ctx->tensors) {
        for (uint64_t i = 0; i < ctx->header.num_tensors; i++) free(ctx->tensors[i].name);
        free(ctx->tensors);
    }
    free(ctx);
}

void gguf_data_dontneed(const struct gguf_context *ctx, const void *p, size_t bytes) {
    if (!ctx || !ctx->map_base || !bytes) return;
    uintptr_t lo = (uintptr_t)ctx->data, hi = lo + ctx->data_size, a = (uintptr_t)p;
    if (a < lo || a + bytes > hi) return;
    uintptr_t pg = (uintptr_t)sysconf(_SC_PAGESIZE);
    uintptr_t b = (a + pg - 1) & ~(pg - 1), e = (a + bytes) & ~(pg - 1);
    if (e <= b) return;
    madvise((void *)b, e - b, MADV_DONTNEED);
    if (ctx->map_fd >= 0)
        posix_fadvise(ctx->map_fd, (off_t)(b - (uintptr_t)ctx->map_base), (off_t)(e - b), POSIX_FADV_DONTNEED);
}

const struct gguf_meta *gguf_find_meta(const struct gguf_context *ctx, const char *key) {
    for (uint64_t i = 0; i < ctx->header.num_meta; i++)
        if (!strcmp(ctx->meta[i].key, key)) return &ctx->meta[i];
    return NULL;
}

const struct gguf_tensor *gguf_find_tensor(const struct gguf_context *ctx, const char *name) {
    for (uint64_t i = 0; i < ctx->header.num_tensors; i++)
        if (!strcmp(ctx->tensors[i].name, name)) return &ctx->tensors[i];
    return NULL;
}

/* integer getters take u32 and i32 interchangeably, the f32 getter only f32
 * (reference src/gguf.c:569-593) */
uint32_t gguf_get_u32(const struct gguf_context *ctx, const char *key, uint32_t fallback) {
    const struct gguf_meta *m = gguf_find_meta(ctx, key);
    if (m && m->type == GGUF_TYPE_UINT32) return m->value.u32;
    if (m && m->type == GGUF_TYPE_INT32) return (uint32_t)m->value.i32;
    return fallback;
}
int32_t gguf_get_i32(const struct gguf_context *ctx, const char *key, int32_t fallback) {
    const struct gguf_meta *m = gguf_find_meta(ctx, key);
    if (m && m->type == GGUF_TYPE_INT32) return m->value.i32;
    if (m && m->type == GGUF_TYPE_UINT32) return (int32_t)m->value.u32;
    return fallback;
}
float gguf_get_f32(const struct gguf_context *ctx, const char *key, float fallback) {
    const struct gguf_meta *m = gguf_find_meta(ctx, key);
    return (m && m->type == GGUF_TYPE_FLOAT32) ? m->value.f32 : fallback;
}
const char *gguf_get_str(const struct gguf_context *ctx, const char *key, const char *fallback) {
    const struct gguf_meta *m = gguf_find_meta(ctx, key);
    return (m && m->type == GGUF_TYPE_STRING) ? m->value.str : fallback;
}

void gguf_dump(const struct gguf_context *ctx) {
    printf("GGUF v%u: %llu tensors, %llu metadata pairs, alignment %zu, data %zu bytes at %zu\n",
           ctx->header.version, (unsigned long long)ctx->header.num_tensors,
           (unsigned long long)ctx->header.num_meta, ctx->alignment, ctx->data_size, ctx->data_offset);
    for (uint64_t i = 0; i < ctx->header.num_meta; i++) {
        const struct gguf_meta *m = &ctx->meta[i];
        printf("  %-56s %s", m->key, gguf_type_name(m->type));
        switch (m->type) {
            case GGUF_TYPE_UINT32: printf(" = %u", m->value.u32); break;
            case GGUF_TYPE_INT32:  printf(" = %d", m->value.i32); break;
            case GGUF_TYPE_FLOAT32: printf(" = %g", m->value.f32); break;
            case GGUF_TYPE_BOOL:   printf(" = %s", m->value.bool_ ? "true" : "false"); break;
            case GGUF_TYPE_STRING: printf(" = \"%.60s\"", m->value.str); break;
            case GGUF_TYPE_ARRAY:  printf("[%s x %llu]", gguf_type_name(m->value.arr.type),
                                          (unsigned long long)m->value.arr.n); break;
            default: break;
        }
        printf("\n");
    }
    for (uint64_t i = 0; i < ctx->header.num_tensors; i++) {
        const struct gguf_tensor *t = &ctx->tensors[i];
        int64_t n = 1;
        printf("  %-40s %-5s [", t->name, ggml_type_name(t->type));
        for (uint32_t d = 0; d < t->n_dims; d++) { n *= (int64_t)t->dims[d]; printf("%s%llu", d ? " x " : "", (unsigned long long)t->dims[d]); }
        printf("] @%llu, %zu bytes\n", (unsigned long long)t->offset, ggml_nbytes(t->type, n));
    }
}

/* ====================  writer  ============================================ */

struct gw_tensor { uint64_t offset; size_t bytes; };
struct lg_gguf_writer {
    int fd;
    uint32_t version, alignment;
    unsigned char *head; size_t head_len, head_cap;      /* metadata section being built */
    unsigned char *tinfo; size_t tinfo_len, tinfo_cap;   /* tensor-info section */
    uint64_t n_meta, n_tensors;
    struct gw_tensor *t; size_t t_cap;
    uint64_t data_len;                                   /* bytes of data section so far */
    unsigned char *map; size_t map_len, data_offset;
};

static int buf_put(unsigned char **b, size_t *len, size_t *cap, const void *src, size_t n) {
    if (*len + n > *cap) {
        size_t nc = *cap ? *cap * 2 : 4096;
        while (nc < *len + n) nc *= 2;
        unsigned char *nb = realloc(*b, nc);
        if (!nb) return -1;
        *b = nb; *cap = nc;
    }
    if (src) memcpy(*b + *len, src, n); else memset(*b + *len, 0, n);
    *len += n;
    return 0;
}
#define HPUT(w, src, n) buf_put(&(w)->head, &(w)->head_len, &(w)->head_cap, (src), (n))
#define TPUT(w, src, n) buf_put(&(w)->tinfo, &(w)->tinfo_len, &(w)->tinfo_cap, (src), (n))

static int put_str(unsigned char **b, size_t *len, size_t *cap, const char *s) {
    uint64_t n = strlen(s);
    return buf_put(b, len, cap, &n, 8) || buf_put(b, len, cap, s, n);
}

struct lg_gguf_writer *lg_gw_open(const char *path, uint32_t version, uint32_t alignment) {
    struct lg_gguf_writer *w = calloc(1, sizeof *w);
    if (!w) return NULL;
    w->fd = open(path, O_RDWR | O_CREAT | O_TRUNC, 0644);
    if (w->fd < 0) { free(w); return NULL; }
    w->version = version ? version : 3;
    w->alignment = alignment ? alignment : 32;
    if (w->alignment != 32) lg_gw_meta_u32(w, "general.alignment", w->alignment);
    return w;
}

static int meta_head(struct lg_gguf_writer *w, const char *key, uint32_t type) {
    w->n_meta++;
    return put_str(&w->head, &w->head_len, &w->head_cap, key) || HPUT(w, &type, 4);
}
int lg_gw_meta_u32(struct lg_gguf_writer *w, const char *key, uint32_t v) {
    return meta_head(w, key, GGUF_TYPE_UINT32) || HPUT(w, &v, 4);
}
int lg_gw_meta_f32(struct lg_gguf_writer *w, const char *key, float v) {
    return meta_head(w, key, GGUF_TYPE_FLOAT32) || HPUT(w, &v, 4);
}
int lg_gw_meta_str(struct lg_gguf_writer *w, const char *key, const char *v) {
    return meta_head(w, key, GGUF_TYPE_STRING) || put_str(&w->head, &w->head_len, &w->head_cap, v);
}
int lg_gw_meta_array(struct lg_gguf_writer *w, const char *key, uint32_t et, uint64_t n, const void *data) {
    size_t es = gguf_type_size(et);
    if (!es) return -1;
    return meta_head(w, key, GGUF_TYPE_ARRAY) || HPUT(w, &et, 4) || HPUT(w, &n, 8) || HPUT(w, data, n * es);
}
int lg_gw_meta_empty_strings(struct lg_gguf_writer *w, const char *key, uint64_t n) {
    uint32_t et = GGUF_TYPE_STRING;
    /* n strings of length zero: n u64 zeros */
    return meta_head(w, key, GGUF_TYPE_ARRAY) || HPUT(w, &et, 4) || HPUT(w, &n, 8) || HPUT(w, NULL, n * 8);
}

int lg_gw_add_tensor(struct lg_gguf_writer *w, const char *name, uint32_t type, uint32_t n_dims, const uint64_t *dims) {
    if (n_dims < 1 || n_dims > 4) return -1;
    int64_t n = 1;
    for (uint32_t d = 0; d < n_dims; d++) n *= (int64_t)dims[d];
    size_t bytes = ggml_nbytes(type, n);
    if (!bytes) return -1;
    if (w->n_tensors == w->t_cap) {
        size_t nc = w->t_cap ? w->t_cap * 2 : 64;
        struct gw_tensor *nt = realloc(w->t, nc * sizeof *nt);
        if (!nt) return -1;
        w->t = nt; w->t_cap = nc;
    }
    uint64_t off = (w->data_len + w->alignment - 1) / w->alignment * w->alignment;
    if (put_str(&w->tinfo, &w->tinfo_len, &w->tinfo_cap, name) || TPUT(w, &n_dims, 4) ||
        TPUT(w, dims, 8 * n_dims) || TPUT(w, &type, 4) || TPUT(w, &off, 8)) return -1;
    w->t[w->n_tensors].offset = off;
    w->t[w->n_tensors].bytes = bytes;
    w->data_len = off + bytes;
    return (int)w->n_tensors++;
}

int lg_gw_commit(struct lg_gguf_writer *w) {
    struct gguf_header h = { GGUF_MAGIC_LE, w->version, w->n_tensors, w->n_meta };
    size_t info = sizeof h + w->head_len + w->tinfo_len;
    w->data_offset = (info + w->alignment - 1) / w->alignment * w->alignment;
    w->map_len = w->data_offset + w->data_len;
    if (ftruncate(w->fd, (off_t)w->map_len) != 0) return -1;
    w->map = mmap(NULL, w->map_len, PROT_READ | PROT_WRITE, MAP_SHARED, w->fd, 0);
    if (w->map == MAP_FAILED) { w->map = NULL; return -1; }
    memcpy(w->map, &h, sizeof h);
    memcpy(w->map + sizeof h, w->head, w->head_len);
    memcpy(w->map + sizeof h + w->head_len, w->tinfo, w->tinfo_len);
    return 0;
}

void *lg_gw_tensor_data(struct lg_gguf_writer *w, int index, size_t *bytes) {
    if (!w->map || index < 0 || (uint64_t)index >= w->n_tensors) return NULL;
    if (bytes) *bytes = w->t[index].bytes;
    return w->map + w->data_offset + w->t[index].offset;
}

int lg_gw_close(struct lg_gguf_writer *w) {
    int rc = 0;
    if (w->map && munmap(w->map, w->map_len) != 0) rc = -1;
    if (close(w->fd) != 0) rc = -1;
    free(w->head); free(w->tinfo); free(w->t); free(w);
    return rc;
}
