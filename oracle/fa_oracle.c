/*
 * CPU oracle for the FlashAttention forward path: TEST INFRASTRUCTURE ONLY.
 * See fa_oracle.h for scope and pinning status.
 *
 * Rounding points follow the reference verifier (reference src/main.cu):
 *   :193  each q*k product is rounded to the storage type, then widened and
 *         summed in fp32, k ascending
 *   :195  score = sum * softmax_scale (fp32)
 *   :200-207 ALiBi  score -= slope * |i-j|
 *   :210-229 causal / window masks set the score to -inf
 *   :232-252 row max, expf(score - max), fp32 sum (j ascending), fp32 divide
 *   :259  p is rounded to the storage type, multiplied by v with the product
 *         rounded to the storage type, widened and summed in fp32, j ascending
 *   :261  the sum is rounded to the storage type
 * Masked keys contribute expf(-inf) = 0 to the sum and a zero product to the
 * output, so skipping them (as the streamed evaluation below does) changes no
 * bit of the result.
 */
#include "fa_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#if defined(__AVX2__) && defined(__F16C__)
#include <immintrin.h>
#define FA_ORACLE_SIMD 1
#else
#define FA_ORACLE_SIMD 0
#endif

/* ------------------------------------------------------------------ */
/* scalar conversions, round-to-nearest-even, written out bit by bit  */
/* ------------------------------------------------------------------ */
static inline uint32_t f32_bits(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static inline float bits_f32(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

uint16_t fa_oracle_f32_to_f16(float x)
{
    uint32_t u = f32_bits(x);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t a = u & 0x7fffffffu;
    if (a >= 0x7f800000u)                       /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (a > 0x7f800000u ? 0x200u : 0u));
    if (a >= 0x477ff000u)                       /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    if (a < 0x38800000u) {                      /* below 2^-14: subnormal half */
        if (a < 0x33000000u) return (uint16_t)sign;   /* < 2^-25 -> 0 (ties to even gives 0 at 2^-25) */
        uint32_t e = a >> 23;                   /* biased exponent, 102..112 */
        uint32_t m = (a & 0x7fffffu) | 0x800000u;
        uint32_t shift = 126u - e;              /* 14..24: m * 2^(e-150) in units of 2^-24 */
        uint32_t q = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1u);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    {
        uint32_t m = a & 0x7fffffu;
        uint32_t e = (a >> 23) - 112u;          /* rebias 127 -> 15 */
        uint32_t q = (e << 10) | (m >> 13);
        uint32_t rem = m & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
}

float fa_oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu;
    uint32_t m = h & 0x3ffu;
    if (e == 0x1fu) return bits_f32(sign | 0x7f800000u | (m << 13));
    if (e == 0) {
        if (m == 0) return bits_f32(sign);
        /* subnormal: m * 2^-24 */
        float v = (float)m * (1.0f / 16777216.0f);
        return sign ? -v : v;
    }
    return bits_f32(sign | ((e + 112u) << 23) | (m << 13));
}

uint16_t fa_oracle_f32_to_bf16(float x)
{
    uint32_t u = f32_bits(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float fa_oracle_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

static inline float widen(uint16_t h, int dtype)
{
    return dtype == FA_ORACLE_F16 ? fa_oracle_f16_to_f32(h) : fa_oracle_bf16_to_f32(h);
}
static inline uint16_t narrow(float x, int dtype)
{
    return dtype == FA_ORACLE_F16 ? fa_oracle_f32_to_f16(x) : fa_oracle_f32_to_bf16(x);
}
/* storage-type product of two storage-type values: the fp32 product of two
 * 11-bit (or 8-bit) significands is exact, so one rounding is all there is. */
static inline float prod_storage(float a, float b, int dtype)
{
    return widen(narrow(a * b, dtype), dtype);
}

static inline int masked(const fa_oracle_cfg *c, int i, int j)
{
    if (c->causal && j > i) return 1;
    if (c->window_left >= 0 && i - j > c->window_left) return 1;
    if (c->window_right >= 0 && j - i > c->window_right) return 1;
    return 0;
}

static int cfg_ok(const fa_oracle_cfg *c)
{
    return c && c->B > 0 && c->H > 0 && c->S > 0 && c->D > 0 &&
           (c->dtype == FA_ORACLE_F16 || c->dtype == FA_ORACLE_BF16) &&
           c->dropout_threshold >= 0 && c->dropout_threshold <= 255;
}

/* ------------------------------------------------------------------ */
/* dropout: a counter-based decision per (head, query, key)            */
/* ------------------------------------------------------------------ */
void fa_oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c[4] = {ctr[0], ctr[1], ctr[2], ctr[3]}, k[2] = {key[0], key[1]};
    for (int round = 0; round < 10; ++round) {
        const uint64_t lo = (uint64_t)0xD2511F53u * c[0], hi = (uint64_t)0xCD9E8D57u * c[2];
        const uint32_t n[4] = {(uint32_t)(hi >> 32) ^ c[1] ^ k[0], (uint32_t)hi, (uint32_t)(lo >> 32) ^ c[3] ^ k[1], (uint32_t)lo};
        memcpy(c, n, sizeof(c));
        k[0] += 0x9E3779B9u;        /* golden-ratio and sqrt(3)-1 Weyl increments */
        k[1] += 0xBB67AE85u;
    }
    memcpy(out, c, sizeof(c));
}

int fa_oracle_dropout_keep(uint64_t seed, int64_t bh, int i, int j, int threshold)
{
    const uint32_t ctr[4] = {(uint32_t)(2 * (j / 32) + (j / 4) % 2), (uint32_t)i, (uint32_t)bh, 0x44524F50u};
    const uint32_t key[2] = {(uint32_t)(seed & 0xffffffffu), (uint32_t)(seed >> 32)};
    uint32_t w[4];
    fa_oracle_philox4x32_10(ctr, key, w);
    const int byte = 4 * ((j % 32) / 8) + j % 4;
    return (int)((w[byte / 4] >> (8 * (byte % 4))) & 255u) >= threshold;
}
/* p after dropout (fp32: one rounding for the division that produced p, one for the product) */
static inline float drop_f32(const fa_oracle_cfg *c, int64_t bh, int i, int j, float p)
{
    if (c->dropout_threshold == 0) return p;
    if (!fa_oracle_dropout_keep(c->dropout_seed, bh, i, j, c->dropout_threshold)) return 0.0f;
    return p * (256.0f / (256.0f - (float)c->dropout_threshold));
}

/* ------------------------------------------------------------------ */
/* literal restatement: reference loop order and S*S buffer            */
/* ------------------------------------------------------------------ */
int fa_oracle_literal(const fa_oracle_cfg *c, const uint16_t *Q, const uint16_t *K,
                      const uint16_t *V, uint16_t *O)
{
    if (!cfg_ok(c) || !Q || !K || !V || !O) return -1;
    const int S = c->S, D = c->D, dt = c->dtype;
    const size_t head = (size_t)S * D;
    float *scores = (float *)malloc((size_t)S * S * sizeof(float));
    if (!scores) return -1;
    for (int b = 0; b < c->B; ++b)
        for (int h = 0; h < c->H; ++h) {
            const size_t base = ((size_t)b * c->H + h) * head;
            const uint16_t *q = Q + base, *k = K + base, *v = V + base;
            uint16_t *o = O + base;
            for (int i = 0; i < S; ++i)
                for (int j = 0; j < S; ++j) {
                    float sum = 0.0f;
                    for (int t = 0; t < D; ++t)
                        sum += prod_storage(widen(q[(size_t)i * D + t], dt),
                                            widen(k[(size_t)j * D + t], dt), dt);
                    scores[(size_t)i * S + j] = sum * c->scale;
                }
            if (c->alibi_slopes) {
                const float slope = c->alibi_slopes[h];
                for (int i = 0; i < S; ++i)
                    for (int j = 0; j < S; ++j)
                        scores[(size_t)i * S + j] -= slope * (float)abs(i - j);
            }
            for (int i = 0; i < S; ++i)
                for (int j = 0; j < S; ++j)
                    if (masked(c, i, j)) scores[(size_t)i * S + j] = -INFINITY;
            for (int i = 0; i < S; ++i) {
                float *row = scores + (size_t)i * S;
                float mx = -INFINITY;
                for (int j = 0; j < S; ++j) mx = fmaxf(mx, row[j]);
                float sum = 0.0f;
                for (int j = 0; j < S; ++j) { row[j] = expf(row[j] - mx); sum += row[j]; }
                for (int j = 0; j < S; ++j) row[j] = drop_f32(c, (int64_t)b * c->H + h, i, j, row[j] / sum);
            }
            for (int i = 0; i < S; ++i)
                for (int t = 0; t < D; ++t) {
                    float sum = 0.0f;
                    for (int j = 0; j < S; ++j)
                        sum += prod_storage(widen(narrow(scores[(size_t)i * S + j], dt), dt),
                                            widen(v[(size_t)j * D + t], dt), dt);
                    o[(size_t)i * D + t] = narrow(sum, dt);
                }
        }
    free(scores);
    return 0;
}

/* ------------------------------------------------------------------ */
/* streamed row evaluation                                             */
/* ------------------------------------------------------------------ */
typedef struct { int64_t row; int64_t pos; } row_ref;
static int row_ref_cmp(const void *a, const void *b)
{
    const row_ref *x = (const row_ref *)a, *y = (const row_ref *)b;
    if (x->row != y->row) return x->row < y->row ? -1 : 1;
    return x->pos < y->pos ? -1 : (x->pos > y->pos);
}

static void visible_range(const fa_oracle_cfg *c, int i, int *lo, int *hi)
{
    int l = 0, h = c->S - 1;
    if (c->causal && h > i) h = i;
    if (c->window_right >= 0 && h > i + c->window_right) h = i + c->window_right;
    if (c->window_left >= 0 && l < i - c->window_left) l = i - c->window_left;
    *lo = l; *hi = h;
}

#if FA_ORACLE_SIMD
static inline __m256 round_storage8(__m256 p, int dtype)
{
    if (dtype == FA_ORACLE_F16)
        return _mm256_cvtph_ps(_mm256_cvtps_ph(p, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
    __m256i u = _mm256_castps_si256(p);
    __m256i lsb = _mm256_and_si256(_mm256_srli_epi32(u, 16), _mm256_set1_epi32(1));
    u = _mm256_add_epi32(u, _mm256_add_epi32(lsb, _mm256_set1_epi32(0x7fff)));
    u = _mm256_and_si256(u, _mm256_set1_epi32((int)0xffff0000u));
    return _mm256_castsi256_ps(u);
}
#endif

/* scores[j - lo] for j in [lo,hi] of one query row; KT is [D][S] fp32 */
static void row_scores(const fa_oracle_cfg *c, const float *qf, const float *KT,
                       int i, int lo, int hi, float slope, float *sc)
{
    const int S = c->S, D = c->D, dt = c->dtype;
    int j = lo;
#if FA_ORACLE_SIMD
    for (; j + 8 <= hi + 1; j += 8) {
        __m256 acc = _mm256_setzero_ps();
        for (int t = 0; t < D; ++t) {
            __m256 p = _mm256_mul_ps(_mm256_set1_ps(qf[t]), _mm256_loadu_ps(KT + (size_t)t * S + j));
            acc = _mm256_add_ps(acc, round_storage8(p, dt));
        }
        acc = _mm256_mul_ps(acc, _mm256_set1_ps(c->scale));
        _mm256_storeu_ps(sc + (j - lo), acc);
    }
#endif
    for (; j <= hi; ++j) {
        float sum = 0.0f;
        for (int t = 0; t < D; ++t) sum += prod_storage(qf[t], KT[(size_t)t * S + j], dt);
        sc[j - lo] = sum * c->scale;
    }
    if (c->alibi_slopes)
        for (j = lo; j <= hi; ++j) sc[j - lo] -= slope * (float)abs(i - j);
}

/* out[t] = sum_j storage(p_j * v_jt), j ascending; Vf is [S][D] fp32 */
static void row_pv(const fa_oracle_cfg *c, const float *p, const float *Vf, int lo, int hi, float *out)
{
    const int D = c->D, dt = c->dtype;
    int t = 0;
#if FA_ORACLE_SIMD
    for (; t + 8 <= D; t += 8) {
        __m256 acc = _mm256_setzero_ps();
        for (int j = lo; j <= hi; ++j) {
            __m256 pr = _mm256_mul_ps(_mm256_set1_ps(p[j - lo]), _mm256_loadu_ps(Vf + (size_t)j * D + t));
            acc = _mm256_add_ps(acc, round_storage8(pr, dt));
        }
        _mm256_storeu_ps(out + t, acc);
    }
#endif
    for (; t < D; ++t) {
        float sum = 0.0f;
        for (int j = lo; j <= hi; ++j) sum += prod_storage(p[j - lo], Vf[(size_t)j * D + t], dt);
        out[t] = sum;
    }
}

int fa_oracle_rows(const fa_oracle_cfg *c, const uint16_t *Q, const uint16_t *K,
                   const uint16_t *V, const int64_t *rows, int64_t nrows,
                   uint16_t *O_rows, float *lse_rows, int nthreads)
{
    if (!cfg_ok(c) || !Q || !K || !V || (nrows > 0 && !rows) || nrows < 0) return -1;
    const int S = c->S, D = c->D, dt = c->dtype;
    const int64_t total = (int64_t)c->B * c->H * S;
    for (int64_t n = 0; n < nrows; ++n)
        if (rows[n] < 0 || rows[n] >= total) return -1;
    if (nrows == 0) return 0;
    if (nthreads < 1) nthreads = 1;

    row_ref *order = (row_ref *)malloc((size_t)nrows * sizeof(row_ref));
    float *KT = (float *)malloc((size_t)S * D * sizeof(float));
    float *Vf = (float *)malloc((size_t)S * D * sizeof(float));
    float *scratch = (float *)malloc((size_t)nthreads * ((size_t)S + 2 * (size_t)D) * sizeof(float));
    if (!order || !KT || !Vf || !scratch) { free(order); free(KT); free(Vf); free(scratch); return -1; }
    for (int64_t n = 0; n < nrows; ++n) { order[n].row = rows[n]; order[n].pos = n; }
    qsort(order, (size_t)nrows, sizeof(row_ref), row_ref_cmp);

    int64_t start = 0;
    while (start < nrows) {
        const int64_t bh = order[start].row / S;
        int64_t end = start;
        while (end < nrows && order[end].row / S == bh) ++end;
        const uint16_t *k = K + (size_t)bh * S * D, *v = V + (size_t)bh * S * D, *q = Q + (size_t)bh * S * D;
        const float slope = c->alibi_slopes ? c->alibi_slopes[bh % c->H] : 0.0f;
        int jmax = 0;
        for (int64_t n = start; n < end; ++n) {
            int lo, hi; visible_range(c, (int)(order[n].row % S), &lo, &hi);
            if (hi > jmax) jmax = hi;
        }
#pragma omp parallel for num_threads(nthreads) schedule(static)
        for (int j = 0; j <= jmax; ++j)
            for (int t = 0; t < D; ++t) {
                KT[(size_t)t * S + j] = widen(k[(size_t)j * D + t], dt);
                Vf[(size_t)j * D + t] = widen(v[(size_t)j * D + t], dt);
            }
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 1)
        for (int64_t n = start; n < end; ++n) {
#ifdef _OPENMP
            const int tid = omp_get_thread_num();
#else
            const int tid = 0;
#endif
            float *sc = scratch + (size_t)tid * ((size_t)S + 2 * (size_t)D);
            float *qf = sc + S, *out = qf + D;
            const int i = (int)(order[n].row % S);
            int lo, hi; visible_range(c, i, &lo, &hi);
            for (int t = 0; t < D; ++t) qf[t] = widen(q[(size_t)i * D + t], dt);
            row_scores(c, qf, KT, i, lo, hi, slope, sc);
            float mx = -INFINITY;
            for (int j = lo; j <= hi; ++j) mx = fmaxf(mx, sc[j - lo]);
            float sum = 0.0f;
            for (int j = lo; j <= hi; ++j) { sc[j - lo] = expf(sc[j - lo] - mx); sum += sc[j - lo]; }
            for (int j = lo; j <= hi; ++j) sc[j - lo] = widen(narrow(drop_f32(c, bh, i, j, sc[j - lo] / sum), dt), dt);
            if (O_rows) {
                row_pv(c, sc, Vf, lo, hi, out);
                for (int t = 0; t < D; ++t) O_rows[(size_t)order[n].pos * D + t] = narrow(out[t], dt);
            }
            if (lse_rows) lse_rows[order[n].pos] = mx + logf(sum);
        }
        start = end;
    }
    free(order); free(KT); free(Vf); free(scratch);
    return 0;
}

int fa_oracle_full(const fa_oracle_cfg *c, const uint16_t *Q, const uint16_t *K,
                   const uint16_t *V, uint16_t *O, float *lse, int nthreads)
{
    if (!cfg_ok(c)) return -1;
    const int64_t total = (int64_t)c->B * c->H * c->S;
    int64_t *rows = (int64_t *)malloc((size_t)total * sizeof(int64_t));
    if (!rows) return -1;
    for (int64_t n = 0; n < total; ++n) rows[n] = n;
    int rc = fa_oracle_rows(c, Q, K, V, rows, total, O, lse, nthreads);
    free(rows);
    return rc;
}

int fa_oracle_rows_f64(const fa_oracle_cfg *c, const uint16_t *Q, const uint16_t *K,
                       const uint16_t *V, const int64_t *rows, int64_t nrows,
                       double *O_rows, double *lse_rows, int nthreads)
{
    if (!cfg_ok(c) || !Q || !K || !V || (nrows > 0 && !rows) || nrows < 0) return -1;
    const int S = c->S, D = c->D, dt = c->dtype;
    const int64_t total = (int64_t)c->B * c->H * S;
    for (int64_t n = 0; n < nrows; ++n)
        if (rows[n] < 0 || rows[n] >= total) return -1;
    if (nthreads < 1) nthreads = 1;
    int bad = 0;
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 1)
    for (int64_t n = 0; n < nrows; ++n) {
        const int64_t bh = rows[n] / S;
        const int i = (int)(rows[n] % S);
        const uint16_t *k = K + (size_t)bh * S * D, *v = V + (size_t)bh * S * D, *q = Q + ((size_t)bh * S + i) * D;
        const double slope = c->alibi_slopes ? (double)c->alibi_slopes[bh % c->H] : 0.0;
        int lo, hi; visible_range(c, i, &lo, &hi);
        double *sc = (double *)malloc(((size_t)(hi - lo + 1) + D) * sizeof(double));
        if (!sc) { bad = 1; continue; }
        double *out = sc + (hi - lo + 1);
        double mx = -INFINITY;
        for (int j = lo; j <= hi; ++j) {
            double s = 0.0;
            for (int t = 0; t < D; ++t) s += (double)widen(q[t], dt) * (double)widen(k[(size_t)j * D + t], dt);
            s = s * (double)c->scale - slope * abs(i - j);
            sc[j - lo] = s;
            if (s > mx) mx = s;
        }
        double sum = 0.0;
        for (int j = lo; j <= hi; ++j) { sc[j - lo] = exp(sc[j - lo] - mx); sum += sc[j - lo]; }
        if (O_rows) {
            for (int t = 0; t < D; ++t) out[t] = 0.0;
            for (int j = lo; j <= hi; ++j) {
                double p = sc[j - lo] / sum;
                if (c->dropout_threshold != 0)
                    p = fa_oracle_dropout_keep(c->dropout_seed, bh, i, j, c->dropout_threshold)
                            ? p * (256.0 / (256.0 - (double)c->dropout_threshold)) : 0.0;
                for (int t = 0; t < D; ++t) out[t] += p * (double)widen(v[(size_t)j * D + t], dt);
            }
            for (int t = 0; t < D; ++t) O_rows[(size_t)n * D + t] = out[t];
        }
        if (lse_rows) lse_rows[n] = mx + log(sum);
        free(sc);
    }
    return bad ? -1 : 0;
}

/* ------------------------------------------------------------------ */
/* gradients, fp64 (the reference has no backward pass: this is the     */
/* mathematics of d/dQ, d/dK, d/dV of O = softmax(scale*Q*K^T + bias)*V */
/* on the storage-type inputs, pinned by finite differences and by      */
/* torch autograd in tests/test_oracle_bwd.py)                          */
/* ------------------------------------------------------------------ */
int fa_oracle_bwd_f64(const fa_oracle_cfg *c, const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                      const uint16_t *dO, double *dQ, double *dK, double *dV, int nthreads)
{
    if (!cfg_ok(c) || !Q || !K || !V || !dO || !dQ || !dK || !dV) return -1;
    /* dropout: O = sum_j m_ij p_ij v_j with m_ij = keep_ij / (1 - p); m enters dV and dP, the softmax Jacobian sees p */
    const double keep_scale = 256.0 / (256.0 - (double)c->dropout_threshold);
    const int S = c->S, D = c->D, dt = c->dtype;
    const int64_t BH = (int64_t)c->B * c->H;
    if (nthreads < 1) nthreads = 1;
    double *lse = (double *)malloc((size_t)BH * S * sizeof(double));
    double *delta = (double *)malloc((size_t)BH * S * sizeof(double));      /* D_i = dO_i . O_i */
    if (!lse || !delta) { free(lse); free(delta); return -1; }
    /* pass over query rows: logsumexp, D, dQ */
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 4)
    for (int64_t row = 0; row < BH * S; ++row) {
        const int64_t bh = row / S;
        const int i = (int)(row % S);
        const uint16_t *q = Q + (size_t)row * D, *k = K + (size_t)bh * S * D, *v = V + (size_t)bh * S * D, *g = dO + (size_t)row * D;
        const double slope = c->alibi_slopes ? (double)c->alibi_slopes[bh % c->H] : 0.0;
        int lo, hi; visible_range(c, i, &lo, &hi);
        const int n = hi - lo + 1;
        double *p = (double *)malloc(((size_t)(n > 0 ? n : 1) + 2 * (size_t)D) * sizeof(double));
        double *o = p + (n > 0 ? n : 1), *dq = o + D;
        double mx = -INFINITY;
        for (int j = lo; j <= hi; ++j) {
            double sc = 0.0;
            for (int t = 0; t < D; ++t) sc += (double)widen(q[t], dt) * (double)widen(k[(size_t)j * D + t], dt);
            sc = sc * (double)c->scale - slope * abs(i - j);
            p[j - lo] = sc;
            if (sc > mx) mx = sc;
        }
        double sum = 0.0;
        for (int j = lo; j <= hi; ++j) { p[j - lo] = exp(p[j - lo] - mx); sum += p[j - lo]; }
        for (int t = 0; t < D; ++t) { o[t] = 0.0; dq[t] = 0.0; }
        for (int j = lo; j <= hi; ++j) {
            p[j - lo] /= sum;
            const double m = c->dropout_threshold == 0 ? 1.0
                : fa_oracle_dropout_keep(c->dropout_seed, bh, i, j, c->dropout_threshold) ? keep_scale : 0.0;
            for (int t = 0; t < D; ++t) o[t] += m * p[j - lo] * (double)widen(v[(size_t)j * D + t], dt);
        }
        double dl = 0.0;
        for (int t = 0; t < D; ++t) dl += (double)widen(g[t], dt) * o[t];
        for (int j = lo; j <= hi; ++j) {
            double dp = 0.0;
            for (int t = 0; t < D; ++t) dp += (double)widen(g[t], dt) * (double)widen(v[(size_t)j * D + t], dt);
            if (c->dropout_threshold != 0)
                dp *= fa_oracle_dropout_keep(c->dropout_seed, bh, i, j, c->dropout_threshold) ? keep_scale : 0.0;
            const double ds = p[j - lo] * (dp - dl) * (double)c->scale;
            for (int t = 0; t < D; ++t) dq[t] += ds * (double)widen(k[(size_t)j * D + t], dt);
        }
        for (int t = 0; t < D; ++t) dQ[(size_t)row * D + t] = dq[t];
        lse[row] = n > 0 ? mx + log(sum) : -INFINITY;
        delta[row] = dl;
        free(p);
    }
    /* pass over key rows: dK, dV from the stored logsumexp and D */
#pragma omp parallel for num_threads(nthreads) schedule(dynamic, 4)
    for (int64_t row = 0; row < BH * S; ++row) {
        const int64_t bh = row / S;
        const int j = (int)(row % S);
        const uint16_t *kj = K + (size_t)row * D, *vj = V + (size_t)row * D;
        const uint16_t *q = Q + (size_t)bh * S * D, *g = dO + (size_t)bh * S * D;
        const double slope = c->alibi_slopes ? (double)c->alibi_slopes[bh % c->H] : 0.0;
        double *acc = (double *)calloc(2 * (size_t)D, sizeof(double));
        double *dk = acc, *dv = acc + D;
        for (int i = 0; i < S; ++i) {
            if (masked(c, i, j)) continue;
            double sc = 0.0, dp = 0.0;
            for (int t = 0; t < D; ++t) {
                sc += (double)widen(q[(size_t)i * D + t], dt) * (double)widen(kj[t], dt);
                dp += (double)widen(g[(size_t)i * D + t], dt) * (double)widen(vj[t], dt);
            }
            sc = sc * (double)c->scale - slope * abs(i - j);
            const double pij = exp(sc - lse[bh * S + i]);
            const double m = c->dropout_threshold == 0 ? 1.0
                : fa_oracle_dropout_keep(c->dropout_seed, bh, i, j, c->dropout_threshold) ? keep_scale : 0.0;
            const double ds = pij * (m * dp - delta[bh * S + i]) * (double)c->scale;
            for (int t = 0; t < D; ++t) {
                dk[t] += ds * (double)widen(q[(size_t)i * D + t], dt);
                dv[t] += m * pij * (double)widen(g[(size_t)i * D + t], dt);
            }
        }
        for (int t = 0; t < D; ++t) { dK[(size_t)row * D + t] = dk[t]; dV[(size_t)row * D + t] = dv[t]; }
        free(acc);
    }
    free(lse); free(delta);
    return 0;
}
