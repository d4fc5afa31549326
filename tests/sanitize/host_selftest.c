/*
 * Host-code self-test meant to be built with -fsanitize=address,undefined (tests/sanitize/Makefile): the seeded
 * input generator (flash-attn-rtx5060_amd/host/fa_inputs.c) and the CPU oracle (oracle/fa_oracle.c), both run
 * on buffers of exactly the documented size so that any access past an end is reported, with odd sizes, more
 * threads than rows, every mask kind, ALiBi, dropout and row subsets that touch the first and the last row.
 * The numerical checks are closed forms (constant V, causal row 0, Philox known answers); the point of the
 * program is what the sanitizers see while they run.  Test infrastructure: nothing in the library uses it.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include "fa_inputs.h"
#include "fa_oracle.h"

static int failures = 0;
#define CHECK(cond, ...) do { if (!(cond)) { ++failures; fprintf(stderr, "FAIL %s:%d: ", __FILE__, __LINE__); \
                                              fprintf(stderr, __VA_ARGS__); fputc('\n', stderr); } } while (0)

static void test_philox_and_conversions(void)
{
    /* Random123 known answers for Philox4x32-10 */
    const uint32_t c0[4] = {0, 0, 0, 0}, k0[2] = {0, 0};
    const uint32_t c1[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu}, k1[2] = {0xffffffffu, 0xffffffffu};
    const uint32_t want0[4] = {0x6627e8d5u, 0xe169c58du, 0xbc57ac4cu, 0x9b00dbd8u};
    const uint32_t want1[4] = {0x408f276du, 0x41c83b0eu, 0xa20bc7c6u, 0x6d5451fdu};
    uint32_t out[4];
    fa_philox4x32_10(c0, k0, out);
    CHECK(!memcmp(out, want0, sizeof(out)), "Philox zero vector (input generator)");
    fa_philox4x32_10(c1, k1, out);
    CHECK(!memcmp(out, want1, sizeof(out)), "Philox ones vector (input generator)");
    fa_oracle_philox4x32_10(c0, k0, out);
    CHECK(!memcmp(out, want0, sizeof(out)), "Philox zero vector (oracle)");
    /* every finite fp16 / bf16 value survives storage -> float -> storage, in both implementations */
    for (uint32_t h = 0; h < 65536u; ++h) {
        const float f = fa_f16_bits_to_f32((uint16_t)h);
        if (f == f) {
            CHECK(fa_f32_to_f16_bits(f) == h, "fp16 round trip of 0x%04x", h);
            CHECK(fa_oracle_f32_to_f16(fa_oracle_f16_to_f32((uint16_t)h)) == h, "oracle fp16 round trip of 0x%04x", h);
        }
        const float b = fa_bf16_bits_to_f32((uint16_t)h);
        if (b == b) {
            CHECK(fa_f32_to_bf16_bits(b) == h, "bf16 round trip of 0x%04x", h);
            CHECK(fa_oracle_f32_to_bf16(fa_oracle_bf16_to_f32((uint16_t)h)) == h, "oracle bf16 round trip of 0x%04x", h);
        }
    }
    /* values the conversions must saturate or keep special */
    const float special[] = {0.0f, -0.0f, 65504.0f, 65520.0f, 1e30f, -1e30f, INFINITY, -INFINITY, NAN, 1e-8f, 5.96e-8f, 6.1e-5f};
    for (size_t i = 0; i < sizeof(special) / sizeof(special[0]); ++i) {
        CHECK(fa_f32_to_f16_bits(special[i]) == fa_oracle_f32_to_f16(special[i]) || special[i] != special[i],
              "fp16 conversions of %g disagree", (double)special[i]);
        CHECK(fa_f32_to_bf16_bits(special[i]) == fa_oracle_f32_to_bf16(special[i]) || special[i] != special[i],
              "bf16 conversions of %g disagree", (double)special[i]);
    }
}

static void test_fill(void)
{
    /* small and odd row counts, more threads than rows (the head dimension is a multiple of four by contract) */
    const struct { uint64_t rows; int d; int threads; } cases[] = {{1, 4, 1}, {1, 12, 8}, {3, 20, 2}, {7, 64, 16}, {33, 36, 3}, {256, 128, 8}};
    for (size_t c = 0; c < sizeof(cases) / sizeof(cases[0]); ++c)
        for (int dtype = 0; dtype < 2; ++dtype) {
            const size_t n = (size_t)cases[c].rows * (size_t)cases[c].d;
            uint16_t *a = malloc(n * sizeof(uint16_t)), *b = malloc(n * sizeof(uint16_t));
            CHECK(a && b, "allocation");
            CHECK(fa_fill_normal(a, cases[c].rows, cases[c].d, dtype, 29, FA_TENSOR_Q, 1.0f, 0.25, 8.0f, cases[c].threads) == 0, "fill");
            CHECK(fa_fill_normal(b, cases[c].rows, cases[c].d, dtype, 29, FA_TENSOR_Q, 1.0f, 0.25, 8.0f, 1) == 0, "fill");
            CHECK(!memcmp(a, b, n * sizeof(uint16_t)), "fill depends on the thread count (rows %llu d %d)", (unsigned long long)cases[c].rows, cases[c].d);
            for (size_t i = 0; i < n; ++i) {
                const uint64_t row = i / (size_t)cases[c].d;
                const float z = fa_input_normal(29, FA_TENSOR_Q, i) * (fa_input_row_selected(29, FA_TENSOR_Q, row, 0.25) ? 8.0f : 1.0f);
                const uint16_t want = dtype ? fa_f32_to_bf16_bits(z) : fa_f32_to_f16_bits(z);
                if (a[i] != want) { CHECK(0, "element %zu of a fill differs from the per-element function", i); break; }
            }
            free(a); free(b);
        }
    uint16_t one;
    CHECK(fa_fill_normal(NULL, 1, 1, 0, 1, FA_TENSOR_K, 1.0f, 0.0, 1.0f, 1) != 0, "NULL destination accepted");
    CHECK(fa_fill_normal(&one, 1, 0, 0, 1, FA_TENSOR_K, 1.0f, 0.0, 1.0f, 1) != 0, "d = 0 accepted");
    CHECK(fa_fill_normal(&one, 1, 3, 0, 1, FA_TENSOR_K, 1.0f, 0.0, 1.0f, 1) != 0, "d = 3 accepted");
    CHECK(fa_fill_normal(&one, 1, 4, 7, 1, FA_TENSOR_K, 1.0f, 0.0, 1.0f, 1) != 0, "dtype 7 accepted");
}

static void test_oracle(void)
{
    const struct { int B, H, S, D, causal, wl, wr, alibi, drop; } cases[] = {
        {1, 1, 1, 8, 0, -1, -1, 0, 0},   {1, 2, 5, 8, 1, -1, -1, 0, 0},    {2, 3, 17, 16, 0, 3, 0, 1, 0},
        {1, 2, 33, 64, 1, 4, -1, 0, 26}, {1, 1, 40, 128, 0, 2, 5, 1, 128}, {1, 4, 64, 64, 1, -1, -1, 1, 0},
    };
    for (size_t c = 0; c < sizeof(cases) / sizeof(cases[0]); ++c)
        for (int dtype = 0; dtype < 2; ++dtype) {
            const int B = cases[c].B, H = cases[c].H, S = cases[c].S, D = cases[c].D;
            const size_t rows = (size_t)B * H * S, n = rows * (size_t)D;
            uint16_t *q = malloc(n * 2), *k = malloc(n * 2), *v = malloc(n * 2), *o = malloc(n * 2), *o2 = malloc(n * 2), *dO = malloc(n * 2);
            float *lse = malloc(rows * sizeof(float)), *slopes = malloc((size_t)H * sizeof(float));
            double *g = malloc(3 * n * sizeof(double));
            CHECK(q && k && v && o && o2 && dO && lse && slopes && g, "allocation");
            fa_fill_normal(q, rows, D, dtype, 5, FA_TENSOR_Q, 1.0f, 0.0, 1.0f, 4);
            fa_fill_normal(k, rows, D, dtype, 5, FA_TENSOR_K, 1.0f, 0.0, 1.0f, 4);
            fa_fill_normal(dO, rows, D, dtype, 6, FA_TENSOR_V, 1.0f, 0.0, 1.0f, 4);
            /* V constant per column: every output row must be that constant, whatever the mask (no dropout) */
            for (size_t i = 0; i < n; ++i) {
                const float val = 0.25f * (float)((int)(i % (size_t)D) - D / 2);
                v[i] = dtype ? fa_f32_to_bf16_bits(val) : fa_f32_to_f16_bits(val);
            }
            for (int h = 0; h < H; ++h) slopes[h] = (h & 1) ? -0.5f / (float)(h + 1) : 0.25f;
            fa_oracle_cfg cfg;
            memset(&cfg, 0, sizeof(cfg));
            cfg.B = B; cfg.H = H; cfg.S = S; cfg.D = D; cfg.dtype = dtype;
            cfg.scale = (float)(1.0 / sqrt((double)D));
            cfg.causal = cases[c].causal; cfg.window_left = cases[c].wl; cfg.window_right = cases[c].wr;
            cfg.alibi_slopes = cases[c].alibi ? slopes : NULL;
            cfg.dropout_threshold = cases[c].drop; cfg.dropout_seed = 48;
            CHECK(fa_oracle_full(&cfg, q, k, v, o, lse, 8) == 0, "fa_oracle_full, case %zu", c);
            CHECK(fa_oracle_full(&cfg, q, k, v, o2, NULL, 1) == 0, "fa_oracle_full, one thread");
            CHECK(!memcmp(o, o2, n * 2), "oracle result depends on the thread count, case %zu", c);
            if (!cases[c].drop)
                for (size_t i = 0; i < n; ++i) {
                    const float got = dtype ? fa_bf16_bits_to_f32(o[i]) : fa_f16_bits_to_f32(o[i]);
                    const float want = dtype ? fa_bf16_bits_to_f32(v[i]) : fa_f16_bits_to_f32(v[i]);
                    if (fabsf(got - want) > (dtype ? 0.13f : 0.017f)) { CHECK(0, "constant V, case %zu element %zu: %g != %g", c, i, (double)got, (double)want); break; }
                }
            CHECK(fa_oracle_literal(&cfg, q, k, v, o2) == 0, "fa_oracle_literal, case %zu", c);
            CHECK(!memcmp(o, o2, n * 2), "literal and streamed evaluation differ, case %zu", c);
            /* row subsets: first row, last row, one in the middle, in descending order, outputs of exactly 3 rows */
            const int64_t pick[3] = {(int64_t)rows - 1, (int64_t)(rows / 2), 0};
            uint16_t *o3 = malloc(3 * (size_t)D * 2);
            float l3[3];
            double *o64 = malloc(3 * (size_t)D * sizeof(double)), l64[3];
            CHECK(o3 && o64, "allocation");
            CHECK(fa_oracle_rows(&cfg, q, k, v, pick, 3, o3, l3, 5) == 0, "fa_oracle_rows, case %zu", c);
            for (int r = 0; r < 3; ++r) {
                CHECK(!memcmp(o3 + (size_t)r * D, o + (size_t)pick[r] * D, (size_t)D * 2), "row subset differs from the whole tensor, case %zu row %d", c, r);
                CHECK(l3[r] == lse[pick[r]] || (l3[r] != l3[r] && lse[pick[r]] != lse[pick[r]]), "logsumexp of a row subset differs, case %zu row %d", c, r);
            }
            CHECK(fa_oracle_rows(&cfg, q, k, v, pick, 3, NULL, NULL, 2) == 0, "fa_oracle_rows without outputs");
            CHECK(fa_oracle_rows_f64(&cfg, q, k, v, pick, 3, o64, l64, 3) == 0, "fa_oracle_rows_f64, case %zu", c);
            if (!cases[c].drop)
                for (int r = 0; r < 3; ++r)
                    CHECK(fabs(l64[r] - (double)l3[r]) < 0.05, "fp64 and faithful logsumexp far apart, case %zu row %d: %g %g", c, r, l64[r], (double)l3[r]);
            CHECK(fa_oracle_bwd_f64(&cfg, q, k, v, dO, g, g + n, g + 2 * n, 4) == 0, "fa_oracle_bwd_f64, case %zu", c);
            for (size_t i = 0; i < 3 * n; ++i)
                if (!isfinite(g[i])) { CHECK(0, "non-finite gradient, case %zu", c); break; }
            /* bad arguments are refused, not dereferenced */
            const int64_t bad_row[1] = {(int64_t)rows};
            CHECK(fa_oracle_rows(&cfg, q, k, v, bad_row, 1, o3, l3, 1) != 0, "row index past the end accepted");
            CHECK(fa_oracle_rows(&cfg, NULL, k, v, pick, 3, o3, l3, 1) != 0, "NULL Q accepted");
            free(q); free(k); free(v); free(o); free(o2); free(dO); free(lse); free(slopes); free(g); free(o3); free(o64);
        }
    /* dropout decisions: threshold 0 keeps everything, a threshold keeps about (256 - t)/256 */
    long kept = 0;
    for (int i = 0; i < 64; ++i)
        for (int j = 0; j < 256; ++j) {
            CHECK(fa_oracle_dropout_keep(48, 3, i, j, 0) == 1, "threshold 0 dropped a key");
            kept += fa_oracle_dropout_keep(48, 3, i, j, 64);
        }
    CHECK(labs(kept - 64 * 256 * 3 / 4) < 400, "dropout keep rate %ld of %d at threshold 64", kept, 64 * 256);
}

int main(void)
{
    test_philox_and_conversions();
    test_fill();
    test_oracle();
    if (failures) { fprintf(stderr, "%d check(s) failed\n", failures); return 1; }
    puts("host self-test passed");
    return 0;
}
