/* Exerciser for a sanitizer build of the C11 host engine: loads each model file
 * named on the command line (path, vocabulary size), prefills sixteen sessions
 * with prompts whose lengths sit on and around the chunk edges, takes batched
 * and single steps, offers two refused inputs, and frees everything in an order
 * that leaves sessions alive while others are destroyed.  Built and run by
 * tests/test_host_sanitize.py with -fsanitize=address,undefined. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "wayruntime/wayruntime.h"

static int run(wr_engine *e, const char *path, uint32_t vocab)
{
    wr_model *m = NULL;
    wr_model_params mp = {0};
    mp.max_context = 1024;
    if (wr_model_load(e, path, &mp, &m) != 0) { printf("load failed %s\n", path); return 1; }
    wr_session *s[16];
    for (int i = 0; i < 16; i++)
        if (wr_session_create(m, NULL, &s[i]) != 0) { printf("session failed\n"); return 1; }
    uint32_t ids[700];
    for (int i = 0; i < 700; i++) ids[i] = (uint32_t)((i * 2654435761u) % vocab);
    /* prompts of several lengths, including chunk edges and one row */
    const int lens[16] = {1, 2, 7, 8, 9, 63, 64, 65, 255, 256, 257, 300, 511, 512, 513, 700};
    for (int i = 0; i < 16; i++) {
        int r = wr_prefill(s[i], ids, (uint32_t)lens[i]);
        if (r != lens[i]) { printf("prefill %d -> %d\n", lens[i], r); return 1; }
    }
    double acc = 0;
    for (int step = 0; step < 6; step++) {
        uint32_t tok[16]; const float *lg[16];
        for (int i = 0; i < 16; i++) tok[i] = (uint32_t)((step * 31 + i * 7) % vocab);
        int n = 1 + (step * 5) % 16;
        if (wr_batch_step((wr_session *const *)s, tok, (uint32_t)n, lg) != n) { printf("batch failed\n"); return 1; }
        for (int i = 0; i < n; i++) acc += lg[i][0] + lg[i][vocab - 1];
        const float *l1 = wr_step(s[15 - (step % 3)], tok[0]);
        if (!l1) { printf("step failed\n"); return 1; }
        acc += l1[vocab / 2];
    }
    /* refused inputs */
    if (wr_step(s[0], vocab) != NULL) { printf("oov accepted\n"); return 1; }
    uint32_t bad[2] = {1, vocab + 3};
    if (wr_prefill(s[0], bad, 2) >= 0) { printf("bad prefill accepted\n"); return 1; }
    for (int i = 0; i < 16; i += 2) wr_session_destroy(s[i]);
    const float *l2 = wr_step(s[1], 3);
    if (!l2) { printf("step after destroy failed\n"); return 1; }
    for (int i = 1; i < 16; i += 2) wr_session_destroy(s[i]);
    wr_model_free(m);
    printf("%s ok acc=%g\n", path, acc); fflush(stdout);
    return 0;
}

int main(int argc, char **argv)
{
    wr_engine *e = NULL;
    wr_engine_config cfg; memset(&cfg, 0, sizeof cfg);
    if (wr_engine_create(&cfg, &e) != 0) { printf("engine failed\n"); return 1; }
    int rc = 0;
    for (int i = 1; i + 1 < argc && !rc; i += 2) rc = run(e, argv[i], (uint32_t)atoi(argv[i + 1]));
    wr_engine_destroy(e);
    return rc;
}
