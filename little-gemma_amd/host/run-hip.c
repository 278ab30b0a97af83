/* run-hip — the reference CLI's generation path on the gfx950 backend, for token ids.
 *
 * The reference's `run` takes text (-p) and a draft-head file (-mtp) and prints text
 * (src/run.c:697-842).  Tokenizer and chat template are outside this build, so run-hip keeps the
 * flags and the loop (prefill, first token, plain or block-LG_MTP_N speculative greedy steps, the
 * same stderr statistics lines) but takes the prompt as token ids and prints token ids:
 *
 *   run-hip -m model.gguf -p 12,7,99,4 [-n 256] [-mtp assistant.gguf [-rounds R] | -mtp drafts.txt | -mtp self]
 *
 * -mtp assistant.gguf drafts with a gemma4-assistant head on the device, like the reference's -mtp
 * (src/run.c:719), after a plain greedy run of the same prompt: the two outputs must be
 * byte-identical (docs/mtp.md:16-19) and the exit status says whether they were.  -rounds R keeps R
 * speculative rounds on the device between host waits (default 8); 0 waits after every draft and
 * every verify step, as the reference's loop does.  -mtp drafts.txt replays a file of draft token
 * ids instead of a head; -mtp self replays the plain run's own output as (perfect) drafts.
 * Output: generated token ids on stdout, one line.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "model.h"
#include "session.h"

static double now_sec(void) {                       /* wall clock, like src/run.c:42-46 */
    struct timespec ts;
    timespec_get(&ts, TIME_UTC);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

static int parse_ids(const char *s, int *out, int cap) {
    int n = 0;
    while (*s && n < cap) {
        char *end;
        long v = strtol(s, &end, 10);
        if (end == s) break;
        out[n++] = (int)v;
        s = end;
        while (*s == ',' || *s == ' ' || *s == '\n') s++;
    }
    return n;
}

int main(int argc, char **argv) {
    const char *model = NULL, *prompt = NULL, *mtp = NULL;
    int n_gen = 256, rounds = 8;
    for (int i = 1; i < argc; i++) {
        if (!strcmp(argv[i], "-m") && i + 1 < argc) model = argv[++i];
        else if (!strcmp(argv[i], "-p") && i + 1 < argc) prompt = argv[++i];
        else if (!strcmp(argv[i], "-mtp") && i + 1 < argc) mtp = argv[++i];
        else if (!strcmp(argv[i], "-n") && i + 1 < argc) n_gen = atoi(argv[++i]);
        else if (!strcmp(argv[i], "-rounds") && i + 1 < argc) rounds = atoi(argv[++i]);
    }
    if (!model || !prompt) {
        printf("Usage: %s -m <model.gguf> -p <id,id,...> [-n N] [-mtp <assistant.gguf> [-rounds R] | -mtp <draft-ids.txt> | -mtp self]\n"
               "       -rounds R: speculative rounds kept on the device between host waits (default 8; 0 = one wait per draft\n"
               "       and per verify step, like the reference's loop)\n"
               "       (built with LG_MTP_N=%d: speculative blocks verify %d tokens per step)\n", argv[0], LG_MTP_N, LG_MTP_N);
        return 1;
    }
    static int ids[8192];
    int n_prompt = parse_ids(prompt, ids, 8192);
    if (n_prompt < 1 || n_gen < 1) { fprintf(stderr, "run-hip: empty prompt\n"); return 1; }
    struct lg_session *s = lg_session_open(model);
    if (!s) { fprintf(stderr, "run-hip: cannot load %s\n", model); return 1; }
    config_print(&lg_session_model(s)->cfg);
    const int max_seq = n_prompt + n_gen + 1;                       /* src/run.c:715 */
    int *emitted = calloc((size_t)n_gen, sizeof(int)), *drafts = NULL, *plain = NULL;
    if (!emitted) return 1;

    if (mtp) {
        drafts = calloc((size_t)n_gen + 64, sizeof(int));
        if (!drafts) return 1;
        const size_t ml = strlen(mtp);
        if (ml > 5 && !strcmp(mtp + ml - 5, ".gguf")) {
            /* a draft-head file, as the reference's -mtp takes (src/run.c:719): plain greedy run
             * first, then the same generation with the head drafting; the outputs must be equal */
            plain = calloc((size_t)n_gen, sizeof(int));
            if (!plain || lg_session_kv(s, max_seq) != 0) return 1;
            int st;
            lg_session_generate(s, ids, n_prompt, n_gen, 1, NULL, plain, &st);
            struct mtp *head = lg_session_mtp_open(s, mtp);
            if (!head) return 1;
            if (lg_session_kv(s, max_seq) != 0) return 1;
            int steps = 0, nd = 0, na = 0;
            double t0 = now_sec();
            int g = rounds > 0 ? lg_session_generate_mtp_rounds(s, head, ids, n_prompt, n_gen, LG_MTP_N, rounds, emitted, &steps, &nd, &na)
                               : lg_session_generate_mtp(s, head, ids, n_prompt, n_gen, LG_MTP_N, emitted, &steps, &nd, &na);
            double dt = now_sec() - t0;
            for (int i = 0; i < g; i++) printf("%s%d", i ? "," : "", emitted[i]);
            printf("\n");
            fprintf(stderr, "gen:    %d tokens in %.2fs (%.2f tok/s)\n", g, dt, g / (dt > 0 ? dt : 1e-9));
            fprintf(stderr, "mtp:    %d steps, %d drafts, %d accepted (%.0f%%), block %d\n", steps, nd, na, nd ? 100.0 * na / nd : 0.0, LG_MTP_N);
            int bad = g != n_gen || memcmp(plain, emitted, (size_t)g * sizeof(int)) != 0;
            fprintf(stderr, "check:  -mtp output %s plain greedy output\n", bad ? "DIFFERS FROM" : "is byte-identical to");
            lg_session_mtp_close(head);
            free(emitted); free(drafts); free(plain);
            lg_session_close(s);
            return bad;
        } else if (!strcmp(mtp, "self")) {
            plain = calloc((size_t)n_gen, sizeof(int));
            if (!plain || lg_session_kv(s, max_seq) != 0) return 1;
            int steps;
            lg_session_generate(s, ids, n_prompt, n_gen, 1, NULL, plain, &steps);
            memcpy(drafts, plain, (size_t)n_gen * sizeof(int));
        } else {
            FILE *f = fopen(mtp, "r");
            if (!f) { perror(mtp); return 1; }
            static char buf[1 << 20];
            size_t got = fread(buf, 1, sizeof buf - 1, f);
            buf[got] = 0;
            fclose(f);
            parse_ids(buf, drafts, n_gen);
        }
    }
    if (lg_session_kv(s, max_seq) != 0) { fprintf(stderr, "run-hip: kvcache_init failed\n"); return 1; }
    int steps = 0;
    double t0 = now_sec();
    int g = lg_session_generate(s, ids, n_prompt, n_gen, mtp ? LG_MTP_N : 1, drafts, emitted, &steps);
    double dt = now_sec() - t0;
    for (int i = 0; i < g; i++) printf("%s%d", i ? "," : "", emitted[i]);
    printf("\n");
    fprintf(stderr, "gen:    %d tokens in %.2fs (%.2f tok/s), prompt %d tokens included\n", g, dt, g / (dt > 0 ? dt : 1e-9), n_prompt);
    if (mtp) {
        int accepted = g - 1 - steps > 0 ? g - 1 - steps : 0;
        fprintf(stderr, "mtp:    %d verify/decode steps for %d tokens (block %d, %.2f tokens per step, %d drafts accepted)\n",
                steps, g, LG_MTP_N, steps ? (double)(g - 1) / steps : 0.0, accepted);
    }
    int rc = 0;
    if (plain) {
        rc = memcmp(plain, emitted, (size_t)g * sizeof(int)) != 0;
        fprintf(stderr, "check:  -mtp output %s plain greedy output\n", rc ? "DIFFERS FROM" : "is byte-identical to");
    }
    free(emitted); free(drafts); free(plain);
    lg_session_close(s);
    return rc;
}
