/* session.c — see session.h. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "session.h"
#include "lg_hip.h"

int lg_model_forward_spec_n(struct model *m, struct kvcache *kv, const int *toks, int rows, int pos, int *out);
lg_hip_model *lg_mtp_device(struct mtp *t, const struct model *m);
void lg_model_release(void);
int lg_model_mtp_rounds(struct mtp *t, const struct model *m, struct kvcache *kv, int token, int pos, int rows,
                        int n_rounds, int *blocks, int *out, int *adv);

struct lg_session { struct gguf_context *ctx; struct model m; struct kvcache kv; int has_kv; };

struct lg_session *lg_session_open(const char *path) {
    struct lg_session *s = calloc(1, sizeof *s);
    if (!s) return NULL;
    s->ctx = load_gguf(path);
    if (!s->ctx || model_init(&s->m, s->ctx) != 0) { free_gguf(s->ctx); free(s); return NULL; }
    return s;
}
void lg_session_close(struct lg_session *s) {
    if (!s) return;
    if (s->has_kv) kvcache_free(&s->kv);
    lg_model_release();               /* the device copy of the weights goes with the model it was made from */
    model_free(&s->m);
    free_gguf(s->ctx);
    free(s);
}
int lg_session_kv(struct lg_session *s, int max_seq) {
    if (s->has_kv) kvcache_free(&s->kv);
    s->has_kv = kvcache_init(&s->kv, &s->m, max_seq) == 0;
    return s->has_kv ? 0 : -1;
}
struct model   *lg_session_model(struct lg_session *s) { return &s->m; }
struct kvcache *lg_session_kvcache(struct lg_session *s) { return s->has_kv ? &s->kv : NULL; }
int lg_session_info(struct lg_session *s, int *out, int cap) {
    const struct config *c = &s->m.cfg;
    const int v[] = { c->n_layer, c->n_embd, c->n_head, c->n_vocab, c->n_embd_per_layer, c->n_kv_start,
                      c->sliding_window, c->n_ff, c->n_head_kv, c->head_dim_swa, c->head_dim_full, c->n_ctx };
    const int n = (int)(sizeof v / sizeof v[0]);
    for (int i = 0; i < n && i < cap; i++) out[i] = v[i];
    return n;
}
int lg_session_layer(struct lg_session *s, int L, int *out4) {
    if (L < 0 || L >= s->m.cfg.n_layer) return -1;
    out4[0] = s->m.is_local[L]; out4[1] = s->m.head_dim[L]; out4[2] = s->m.n_head_kv[L]; out4[3] = s->m.ffn_len[L];
    return 0;
}
void lg_session_prefill(struct lg_session *s, const int *t, int n, int pos0) { model_prefill(&s->m, &s->kv, t, n, pos0); }
int  lg_session_forward_next(struct lg_session *s, int token, int pos) { return model_forward_next(&s->m, &s->kv, token, pos); }
void lg_session_forward(struct lg_session *s, int token, int pos, float *logits) { model_forward(&s->m, &s->kv, token, pos, logits); }
int  lg_session_forward_spec(struct lg_session *s, const int *toks, int rows, int pos, int *out) {
    return lg_model_forward_spec_n(&s->m, &s->kv, toks, rows, pos, out);
}

/* The generation loop of the reference (src/run.c:737-768) on token ids: prefill all but the last
 * prompt token, pick the first token from the last one, then plain or block-speculative greedy
 * steps; the speculative path falls back to plain steps when a block would not fit the cache
 * (src/run.c:752) and never emits past n_gen. */
int lg_session_generate(struct lg_session *s, const int *prompt, int n_prompt, int n_gen, int rows,
                        const int *drafts, int *emitted, int *steps) {
    if (n_prompt < 1 || !s->has_kv) return -1;
    model_prefill(&s->m, &s->kv, prompt, n_prompt - 1, 0);
    int pos = n_prompt - 1, g = 0, n_steps = 0;
    int best = model_forward_next(&s->m, &s->kv, prompt[n_prompt - 1], pos++);
    while (g < n_gen) {
        emitted[g++] = best;
        if (rows < 2 || g >= n_gen || pos + rows - 1 >= s->kv.max_seq) {
            if (g < n_gen) { best = model_forward_next(&s->m, &s->kv, best, pos++); n_steps++; }
            continue;
        }
        int toks[16], out[16];
        toks[0] = best;
        for (int j = 1; j < rows; j++) toks[j] = drafts ? drafts[g - 1 + j] : toks[j - 1];
        int adv = lg_model_forward_spec_n(&s->m, &s->kv, toks, rows, pos, out);
        n_steps++;
        pos += adv;
        for (int e = 1; e < adv && g < n_gen; e++) emitted[g++] = toks[e];
        best = out[adv - 1];
    }
    if (steps) *steps = n_steps;
    return g;
}

/* ---- with a draft head ------------------------------------------------------------------------ */
struct mtp *lg_session_mtp_open(struct lg_session *s, const char *path) { return mtp_open(path, &s->m); }
void lg_session_mtp_close(struct mtp *t) { mtp_free(t); }
int  lg_session_mtp_draft(struct lg_session *s, struct mtp *t, int token, int pos, int chain) {
    return chain ? mtp_draft_chain(t, &s->m, &s->kv, token, pos) : mtp_draft(t, &s->m, &s->kv, token, pos);
}
int  lg_session_mtp_hidden(struct lg_session *s, struct mtp *t, float *dst) {
    lg_hip_model *d = lg_mtp_device(t, &s->m);
    return d ? lg_hip_get_hidden(d, dst) : -1;
}
int  lg_session_mtp_logits(struct lg_session *s, struct mtp *t, int on, float *dst) {
    lg_hip_model *d = lg_mtp_device(t, &s->m);
    if (!d) return -1;
    if (!dst) return lg_hip_set_option(d, "store_logits", on);
    return lg_hip_get_logits(d, 0, dst);
}

/* The reference's speculative loop (src/run.c:54-71 mtp_step inside :737-768): the head drafts
 * toks[1] from the target's hidden, chains toks[2..] on its own, the target verifies the block.
 * A draft that is unavailable (-1) is padded with the previous token. */
int lg_session_generate_mtp(struct lg_session *s, struct mtp *t, const int *prompt, int n_prompt, int n_gen, int rows,
                            int *emitted, int *steps, int *n_draft, int *n_accept) {
    if (n_prompt < 1 || !s->has_kv || rows < 2 || rows > 16) return -1;
    model_prefill(&s->m, &s->kv, prompt, n_prompt - 1, 0);
    int pos = n_prompt - 1, g = 0, n_steps = 0, nd = 0, na = 0;
    int best = model_forward_next(&s->m, &s->kv, prompt[n_prompt - 1], pos++);
    while (g < n_gen) {
        emitted[g++] = best;
        if (g >= n_gen) break;
        if (pos + rows - 1 >= s->kv.max_seq) { best = model_forward_next(&s->m, &s->kv, best, pos++); n_steps++; continue; }
        int toks[16], out[16];
        toks[0] = best;
        int d = mtp_draft(t, &s->m, &s->kv, best, pos);
        toks[1] = d >= 0 ? d : best;
        for (int j = 2; j < rows; j++) {
            int dj = mtp_draft_chain(t, &s->m, &s->kv, toks[j - 1], pos + j - 1);
            toks[j] = dj >= 0 ? dj : toks[j - 1];
        }
        int adv = lg_model_forward_spec_n(&s->m, &s->kv, toks, rows, pos, out);
        n_steps++; nd += rows - 1; na += adv - 1;
        pos += adv;
        for (int e = 1; e < adv && g < n_gen; e++) emitted[g++] = toks[e];
        best = out[adv - 1];
    }
    if (steps) *steps = n_steps;
    if (n_draft) *n_draft = nd;
    if (n_accept) *n_accept = na;
    return g;
}

/* The same loop with `batch` rounds at a time kept on the device (drafts, verify, accept and the next chosen token
 * never visit the host inside a batch).  Tokens, step and draft counts are those of lg_session_generate_mtp as long
 * as both run whole rounds; near the end of the cache, or when the head cannot chain, the rest of the generation
 * goes through the host-driven rounds.  A batch may run rounds past n_gen: their tokens are dropped and not counted. */
int lg_session_generate_mtp_rounds(struct lg_session *s, struct mtp *t, const int *prompt, int n_prompt, int n_gen, int rows,
                                   int batch, int *emitted, int *steps, int *n_draft, int *n_accept) {
    if (n_prompt < 1 || !s->has_kv || rows < 2 || rows > 16 || batch < 1) return -1;
    int *blocks = malloc((size_t)batch * rows * 2 * sizeof(int)), *adv = malloc((size_t)batch * sizeof(int));
    if (!blocks || !adv) { free(blocks); free(adv); return -1; }
    int *out = blocks + (size_t)batch * rows;
    model_prefill(&s->m, &s->kv, prompt, n_prompt - 1, 0);
    int pos = n_prompt - 1, g = 0, n_steps = 0, nd = 0, na = 0, on_device = 1;
    int best = model_forward_next(&s->m, &s->kv, prompt[n_prompt - 1], pos++);
    while (g < n_gen) {
        emitted[g++] = best;
        if (g >= n_gen) break;
        /* rounds still wanted: each emits at least one token; rounds that fit: each may take `rows` positions */
        int want = n_gen - g < batch ? n_gen - g : batch;
        int fit = (s->kv.max_seq - pos) / rows;
        int n = want < fit ? want : fit;
        if (on_device && n >= 1) {
            if (lg_model_mtp_rounds(t, &s->m, &s->kv, best, pos, rows, n, blocks, out, adv) == 0) {
                for (int r = 0; r < n && g < n_gen; r++) {
                    const int *toks = blocks + (size_t)r * rows, a = adv[r];
                    if (r > 0) emitted[g++] = toks[0];              /* the chosen token of a later round */
                    if (g >= n_gen) break;                          /* that round's drafts are past the end: not counted */
                    n_steps++; nd += rows - 1; na += a - 1;
                    pos += a;
                    for (int e = 1; e < a && g < n_gen; e++) emitted[g++] = toks[e];
                    best = out[(size_t)r * rows + a - 1];
                }
                if (g >= n_gen) break;
                continue;                                           /* `best` opens the next batch */
            }
            on_device = 0;                                          /* refused: host-driven rounds from here on */
        }
        if (pos + rows - 1 >= s->kv.max_seq) { best = model_forward_next(&s->m, &s->kv, best, pos++); n_steps++; continue; }
        int toks[16], o[16];
        toks[0] = best;
        int d = mtp_draft(t, &s->m, &s->kv, best, pos);
        toks[1] = d >= 0 ? d : best;
        for (int j = 2; j < rows; j++) {
            int dj = mtp_draft_chain(t, &s->m, &s->kv, toks[j - 1], pos + j - 1);
            toks[j] = dj >= 0 ? dj : toks[j - 1];
        }
        int a = lg_model_forward_spec_n(&s->m, &s->kv, toks, rows, pos, o);
        n_steps++; nd += rows - 1; na += a - 1;
        pos += a;
        for (int e = 1; e < a && g < n_gen; e++) emitted[g++] = toks[e];
        best = o[a - 1];
    }
    free(blocks); free(adv);
    if (steps) *steps = n_steps;
    if (n_draft) *n_draft = nd;
    if (n_accept) *n_accept = na;
    return g;
}
