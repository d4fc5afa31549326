/*
 * Plain-C host harness: the role of the reference's main()
 * (reference src/main.cu:21-132).  It names the problem, generates seeded
 * inputs on the host, moves them to the GPU, runs the forward operator, times
 * it and reports.  It includes no HIP header: everything on the device goes
 * through the C ABI of libfa_fwd_gfx950.so (include/fa_fwd.h).
 *
 * Differences from the reference harness, on purpose:
 *   - shape and flags come from argv instead of edited locals (main.cu:22-32);
 *   - inputs are N(0, sigma^2) from a counter-based generator, not
 *     std::default_random_engine (main.cu:69-81);
 *   - timing is hipEvents around warmed-up launches only, not one cold launch
 *     including set-up (flash_forward.h:646-664);
 *   - the result is written to files (--dump) for an external checker instead
 *     of being verified in-process (main.cu:103-108).
 *
 * usage: fa_harness [--config c1..c5] [--B n --N n --S n --d n] [--bf16]
 *                   [--causal] [--window-left n] [--window-right n]
 *                   [--scale x] [--seed n] [--sigma x] [--iters n] [--warmup n]
 *                   [--threads n] [--dump prefix] [--no-lse] [--backward]
 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "fa_fwd.h"
#include "fa_bwd.h"
#include "fa_inputs.h"

#define PEAK_TFLOPS 2516.6 /* 256 CU x 4096 FLOP/clk x 2.4 GHz, dense fp16 = bf16 */

typedef struct {
    int B, N, S, d, bf16, causal, wl, wr, iters, warmup, threads, lse, alibi;
    unsigned long long seed;
    float sigma, scale, dropout;
    double row_fraction;
    float row_mult;
    const char *dump;
    int backward;       /* also run fa_bwd on a seeded dO (the reference has no backward pass) */
    const char *name;
} cfg_t;

static int set_named(cfg_t *c, const char *name)
{
    c->name = name;
    c->wl = -1; c->wr = -1; c->causal = 0; c->bf16 = 0; c->sigma = 1.0f; c->row_fraction = 0.0; c->row_mult = 1.0f;
    if (!strcmp(name, "c1")) { c->B = 1; c->N = 4; c->S = 256; c->d = 64; c->seed = 26 + 1; }
    else if (!strcmp(name, "c2")) { c->B = 4; c->N = 16; c->S = 2048; c->d = 64; c->causal = 1; c->seed = 26 + 2; }
    else if (!strcmp(name, "c3")) { c->B = 2; c->N = 32; c->S = 8192; c->d = 128; c->causal = 1; c->seed = 26 + 3; }
    else if (!strcmp(name, "c4")) { c->B = 1; c->N = 32; c->S = 16384; c->d = 128; c->bf16 = 1; c->causal = 1; c->wl = 1024; c->seed = 26 + 4; }
    else if (!strcmp(name, "c5")) { c->B = 1; c->N = 64; c->S = 32768; c->d = 128; c->causal = 1; c->sigma = 0.5f; c->row_fraction = 0.01; c->row_mult = 8.0f; c->seed = 26 + 5; }
    else return -1;
    c->scale = (float)(1.0 / sqrt((double)c->d));
    return 0;
}

static int check(int st, const char *what)
{
    if (st == FA_OK) return 0;
    fprintf(stderr, "fa_harness: %s failed: %s", what, fa_strerror(st));
    if (st == FA_ERR_DEVICE) fprintf(stderr, " (%s)", fa_last_device_error());
    fprintf(stderr, "\n");
    return 1;
}

static int dump_file(const char *prefix, const char *suffix, const void *data, size_t bytes)
{
    char path[1024];
    snprintf(path, sizeof(path), "%s.%s", prefix, suffix);
    FILE *f = fopen(path, "wb");
    if (!f) { perror(path); return 1; }
    const size_t n = fwrite(data, 1, bytes, f);
    fclose(f);
    return n != bytes;
}

static int cmp_float(const void *a, const void *b)
{
    const float x = *(const float *)a, y = *(const float *)b;
    return x < y ? -1 : x > y;
}

int main(int argc, char **argv)
{
    cfg_t c;
    memset(&c, 0, sizeof(c));
    set_named(&c, "c1");
    c.iters = 20; c.warmup = 3; c.threads = 8; c.lse = 1;
    int scale_given = 0;
    for (int i = 1; i < argc; ++i) {
        const char *a = argv[i];
        const char *v = (i + 1 < argc) ? argv[i + 1] : NULL;
#define NEED_VALUE() do { if (!v) { fprintf(stderr, "%s needs a value\n", a); return 2; } ++i; } while (0)
        if (!strcmp(a, "--config")) { NEED_VALUE(); if (set_named(&c, v)) { fprintf(stderr, "unknown config %s\n", v); return 2; } scale_given = 0; }
        else if (!strcmp(a, "--B")) { NEED_VALUE(); c.B = atoi(v); c.name = "custom"; }
        else if (!strcmp(a, "--N")) { NEED_VALUE(); c.N = atoi(v); c.name = "custom"; }
        else if (!strcmp(a, "--S")) { NEED_VALUE(); c.S = atoi(v); c.name = "custom"; }
        else if (!strcmp(a, "--d")) { NEED_VALUE(); c.d = atoi(v); c.name = "custom"; }
        else if (!strcmp(a, "--bf16")) c.bf16 = 1;
        else if (!strcmp(a, "--causal")) c.causal = 1;
        else if (!strcmp(a, "--window-left")) { NEED_VALUE(); c.wl = atoi(v); }
        else if (!strcmp(a, "--window-right")) { NEED_VALUE(); c.wr = atoi(v); }
        else if (!strcmp(a, "--scale")) { NEED_VALUE(); c.scale = (float)atof(v); scale_given = 1; }
        else if (!strcmp(a, "--seed")) { NEED_VALUE(); c.seed = strtoull(v, NULL, 10); }
        else if (!strcmp(a, "--sigma")) { NEED_VALUE(); c.sigma = (float)atof(v); }
        else if (!strcmp(a, "--iters")) { NEED_VALUE(); c.iters = atoi(v); }
        else if (!strcmp(a, "--warmup")) { NEED_VALUE(); c.warmup = atoi(v); }
        else if (!strcmp(a, "--threads")) { NEED_VALUE(); c.threads = atoi(v); }
        else if (!strcmp(a, "--dump")) { NEED_VALUE(); c.dump = v; }
        else if (!strcmp(a, "--no-lse")) c.lse = 0;
        else if (!strcmp(a, "--backward")) c.backward = 1;
        else if (!strcmp(a, "--alibi")) c.alibi = 1;
        else if (!strcmp(a, "--dropout")) { NEED_VALUE(); c.dropout = (float)atof(v); }
        else { fprintf(stderr, "unknown argument %s\n", a); return 2; }
    }
    if (!scale_given && c.d > 0) c.scale = (float)(1.0 / sqrt((double)c.d));
    if (c.iters < 1) c.iters = 1;
    if (c.warmup < 0) c.warmup = 0;

    if (fa_dev_count() < 1) { fprintf(stderr, "fa_harness: %s\n", fa_strerror(FA_ERR_NO_DEVICE)); return 3; }
    char devname[128] = "";
    int cus = 0, khz = 0;
    if (check(fa_dev_name(devname, sizeof(devname), &cus, &khz), "device query")) return 3;

    const size_t rows = (size_t)c.B * c.N * c.S;
    const size_t elems = rows * (size_t)c.d, bytes = elems * 2;
    uint16_t *hq = malloc(bytes), *hk = malloc(bytes), *hv = malloc(bytes), *ho = malloc(bytes);
    float *hl = malloc(rows * sizeof(float));
    if (!hq || !hk || !hv || !ho || !hl) { fprintf(stderr, "host allocation failed\n"); return 1; }
    if (fa_fill_normal(hq, rows, c.d, c.bf16, c.seed, FA_TENSOR_Q, c.sigma, c.row_fraction, c.row_mult, c.threads) ||
        fa_fill_normal(hk, rows, c.d, c.bf16, c.seed, FA_TENSOR_K, c.sigma, 0.0, 1.0f, c.threads) ||
        fa_fill_normal(hv, rows, c.d, c.bf16, c.seed, FA_TENSOR_V, c.sigma, 0.0, 1.0f, c.threads)) {
        fprintf(stderr, "input generation failed\n");
        return 1;
    }

    void *dq = NULL, *dk = NULL, *dv = NULL, *dO = NULL, *dl = NULL;
    if (check(fa_dev_malloc(&dq, bytes), "alloc Q") || check(fa_dev_malloc(&dk, bytes), "alloc K") ||
        check(fa_dev_malloc(&dv, bytes), "alloc V") || check(fa_dev_malloc(&dO, bytes), "alloc O") ||
        check(fa_dev_malloc(&dl, rows * sizeof(float)), "alloc LSE")) return 1;
    if (check(fa_dev_h2d(dq, hq, bytes), "H2D Q") || check(fa_dev_h2d(dk, hk, bytes), "H2D K") ||
        check(fa_dev_h2d(dv, hv, bytes), "H2D V") || check(fa_dev_memset(dO, 0xff, bytes), "poison O")) return 1;

    fa_fwd_params p;
    memset(&p, 0, sizeof(p));
    p.Q = dq; p.K = dk; p.V = dv; p.O = dO; p.L = c.lse ? (float *)dl : NULL;
    p.B = c.B; p.N = c.N; p.S = c.S; p.d = c.d;
    p.softmax_scale = c.scale;
    p.window_size_left = c.wl; p.window_size_right = c.wr;
    p.dtype = c.bf16 ? FA_DTYPE_BF16 : FA_DTYPE_F16;
    p.is_causal = c.causal;
    p.dropout_prob = c.dropout;      /* main.cu:26,30 (dropout, dropout_prob) ... */
    p.seed = 48;                     /* ... with the seed main() gives its curand states, main.cu:93 */
    float *hs = NULL;
    void *ds = NULL;
    if (c.alibi) {      /* the slopes of main.cu:36-45: -2^(-8/N * (h+1)), copied to the device */
        hs = malloc((size_t)c.N * sizeof(float));
        if (!hs) { fprintf(stderr, "host allocation failed\n"); return 1; }
        for (int h = 0; h < c.N; ++h) hs[h] = (float)-pow(2.0, -8.0 / c.N * (h + 1));
        if (check(fa_dev_malloc(&ds, (size_t)c.N * sizeof(float)), "alloc slopes") ||
            check(fa_dev_h2d(ds, hs, (size_t)c.N * sizeof(float)), "H2D slopes")) return 1;
        p.alibi_slopes_ptr = ds;
    }

    for (int i = 0; i < c.warmup; ++i)
        if (check(fa_fwd(&p, NULL), "warm-up launch")) return 1;
    if (check(fa_dev_sync(), "sync")) return 1;

    float *ms = malloc((size_t)c.iters * sizeof(float));
    void *e0 = NULL, *e1 = NULL;
    if (!ms || check(fa_event_create(&e0), "event") || check(fa_event_create(&e1), "event")) return 1;
    for (int i = 0; i < c.iters; ++i) {
        if (check(fa_event_record(e0, NULL), "record") || check(fa_fwd(&p, NULL), "launch") ||
            check(fa_event_record(e1, NULL), "record") || check(fa_event_sync(e1), "event sync") ||
            check(fa_event_elapsed_ms(e0, e1, &ms[i]), "elapsed")) return 1;
    }
    if (check(fa_dev_d2h(ho, dO, bytes), "D2H O")) return 1;
    if (c.lse && check(fa_dev_d2h(hl, dl, rows * sizeof(float)), "D2H LSE")) return 1;

    qsort(ms, (size_t)c.iters, sizeof(float), cmp_float);
    const double med = ms[c.iters / 2], best = ms[0];
    const double flops = fa_algorithmic_flops(c.B, c.N, c.S, c.d, c.causal, c.wl, c.wr);
    size_t bad = 0;
    for (size_t i = 0; i < elems; ++i) {
        const float x = c.bf16 ? fa_bf16_bits_to_f32(ho[i]) : fa_f16_bits_to_f32(ho[i]);
        if (!isfinite(x)) ++bad;                      /* main.cu:149 rejects NaN/Inf the same way */
    }
    printf("{\"config\": \"%s\", \"device\": \"%s\", \"compute_units\": %d, \"B\": %d, \"N\": %d, \"S\": %d, \"d\": %d, "
           "\"dtype\": \"%s\", \"causal\": %d, \"window_left\": %d, \"window_right\": %d, \"alibi\": %d, \"dropout\": %.6g, \"scale\": %.9g, \"seed\": %llu, "
           "\"iters\": %d, \"ms_median\": %.6f, \"ms_min\": %.6f, \"algorithmic_flops\": %.6e, "
           "\"tflops_median\": %.3f, \"tflops_best\": %.3f, \"peak_tflops\": %.1f, \"frac_of_peak_median\": %.4f, "
           "\"nonfinite_outputs\": %zu}\n",
           c.name, devname, cus, c.B, c.N, c.S, c.d, c.bf16 ? "bf16" : "fp16", c.causal, c.wl, c.wr, c.alibi, (double)c.dropout, (double)c.scale,
           c.seed, c.iters, med, best, flops, flops / med / 1e9, flops / best / 1e9, PEAK_TFLOPS,
           flops / med / 1e9 / PEAK_TFLOPS, bad);

    int rc = bad ? 4 : 0;
    uint16_t *hg[4] = {NULL, NULL, NULL, NULL};      /* dO, dQ, dK, dV on the host */
    if (c.backward) {
        /* gradients of sum(dO * O) through fa_bwd, with dO from the same generator (tensor slot of Q, seed + 1000):
           a second JSON line; the forward pass above has left O and the logsumexp on the device */
        if (!c.lse) { fprintf(stderr, "--backward needs the logsumexp (drop --no-lse)\n"); return 2; }
        /* fa_bwd recomputes P from exact scores: hand it the O and logsumexp of a forward pass whose first rows
           use exact products too (the default recomputes a causal head's first 32 rows in the CPU verifier's
           rounded-product arithmetic, which is what the check of the forward output above wants) */
        p.exact_first_rows = 1;
        if (check(fa_fwd(&p, NULL), "forward launch for the backward pass") || check(fa_dev_sync(), "sync")) return 1;
        void *dg[4] = {NULL, NULL, NULL, NULL}, *ws = NULL;
        for (int t = 0; t < 4; ++t) {
            hg[t] = malloc(bytes);
            if (!hg[t] || check(fa_dev_malloc(&dg[t], bytes), "alloc gradient")) return 1;
        }
        if (fa_fill_normal(hg[0], rows, c.d, c.bf16, c.seed + 1000, FA_TENSOR_Q, 1.0f, 0.0, 1.0f, c.threads) ||
            check(fa_dev_h2d(dg[0], hg[0], bytes), "H2D dO")) return 1;
        fa_bwd_params b;
        memset(&b, 0, sizeof(b));
        b.Q = dq; b.K = dk; b.V = dv; b.O = dO; b.dO = dg[0]; b.L = (const float *)dl;
        b.dQ = dg[1]; b.dK = dg[2]; b.dV = dg[3];
        b.B = c.B; b.N = c.N; b.S = c.S; b.d = c.d;
        b.softmax_scale = c.scale;
        b.window_size_left = c.wl; b.window_size_right = c.wr;
        b.dtype = p.dtype; b.is_causal = c.causal;
        b.alibi_slopes_ptr = p.alibi_slopes_ptr;
        b.dropout_prob = p.dropout_prob; b.seed = p.seed;
        /* the smallest workspace that selects the five-product form (the dS blocks of a chunk of heads), where the
           problem has that form and the device the memory; else the small one (seven products) */
        b.workspace_bytes = fa_bwd_min_fast_workspace_bytes(&b);
        if (b.workspace_bytes == 0 || fa_dev_malloc(&ws, (size_t)b.workspace_bytes) != FA_OK) {
            b.workspace_bytes = fa_bwd_workspace_bytes(&b);
            if (check(fa_dev_malloc(&ws, (size_t)b.workspace_bytes), "alloc workspace")) return 1;
        }
        b.workspace = ws;
        for (int i = 0; i < c.warmup; ++i)
            if (check(fa_bwd(&b, NULL), "backward warm-up launch")) return 1;
        if (check(fa_dev_sync(), "sync")) return 1;
        for (int i = 0; i < c.iters; ++i) {
            if (check(fa_event_record(e0, NULL), "record") || check(fa_bwd(&b, NULL), "backward launch") ||
                check(fa_event_record(e1, NULL), "record") || check(fa_event_sync(e1), "event sync") ||
                check(fa_event_elapsed_ms(e0, e1, &ms[i]), "elapsed")) return 1;
        }
        size_t bad_g = 0;
        for (int t = 1; t < 4; ++t) {
            if (check(fa_dev_d2h(hg[t], dg[t], bytes), "D2H gradient")) return 1;
            for (size_t i = 0; i < elems; ++i) {
                const float x = c.bf16 ? fa_bf16_bits_to_f32(hg[t][i]) : fa_f16_bits_to_f32(hg[t][i]);
                if (!isfinite(x)) ++bad_g;
            }
        }
        qsort(ms, (size_t)c.iters, sizeof(float), cmp_float);
        const double bmed = ms[c.iters / 2], bbest = ms[0];
        const double bflops = fa_bwd_algorithmic_flops(c.B, c.N, c.S, c.d, c.causal, c.wl, c.wr);
        printf("{\"config\": \"%s backward\", \"iters\": %d, \"ms_median\": %.6f, \"ms_min\": %.6f, \"algorithmic_flops\": %.6e, "
               "\"tflops_median\": %.3f, \"tflops_best\": %.3f, \"frac_of_peak_median\": %.4f, \"nonfinite_gradients\": %zu, "
               "\"workspace_bytes\": %llu}\n",
               c.name, c.iters, bmed, bbest, bflops, bflops / bmed / 1e9, bflops / bbest / 1e9, bflops / bmed / 1e9 / PEAK_TFLOPS, bad_g,
               b.workspace_bytes);
        if (bad_g) rc |= 4;
        for (int t = 0; t < 4; ++t) fa_dev_free(dg[t]);
        fa_dev_free(ws);
    }
    if (c.dump) {
        rc |= dump_file(c.dump, "q.bin", hq, bytes) | dump_file(c.dump, "k.bin", hk, bytes) |
              dump_file(c.dump, "v.bin", hv, bytes) | dump_file(c.dump, "o.bin", ho, bytes);
        if (c.lse) rc |= dump_file(c.dump, "lse.bin", hl, rows * sizeof(float));
        if (c.alibi) rc |= dump_file(c.dump, "slopes.bin", hs, (size_t)c.N * sizeof(float));
        if (c.backward)
            rc |= dump_file(c.dump, "do.bin", hg[0], bytes) | dump_file(c.dump, "dq.bin", hg[1], bytes) |
                  dump_file(c.dump, "dk.bin", hg[2], bytes) | dump_file(c.dump, "dv.bin", hg[3], bytes);
    }
    for (int t = 0; t < 4; ++t) free(hg[t]);
    fa_event_destroy(e0); fa_event_destroy(e1);
    fa_dev_free(dq); fa_dev_free(dk); fa_dev_free(dv); fa_dev_free(dO); fa_dev_free(dl);
    if (ds) fa_dev_free(ds);
    free(hs);
    free(hq); free(hk); free(hv); free(ho); free(hl); free(ms);
    return rc;
}
