/* Seeded counter-based input generator; see fa_inputs.h. */
#include "fa_inputs.h"

#include <math.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

void fa_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4])
{
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int round = 0; round < 10; ++round) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

static uint32_t bits_of(float x) { uint32_t u; memcpy(&u, &x, 4); return u; }
static float float_of(uint32_t u) { float x; memcpy(&x, &u, 4); return x; }

uint16_t fa_f32_to_f16_bits(float x)
{
    const uint32_t u = bits_of(x), sign = (u >> 16) & 0x8000u, a = u & 0x7fffffffu;
    if (a >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (a > 0x7f800000u ? 0x200u : 0u));
    if (a >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
    if (a < 0x38800000u) {
        if (a < 0x33000000u) return (uint16_t)sign;
        const uint32_t shift = 126u - (a >> 23);
        const uint32_t m = (a & 0x7fffffu) | 0x800000u;
        uint32_t q = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1u), halfway = 1u << (shift - 1u);
        if (rem > halfway || (rem == halfway && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t q = (((a >> 23) - 112u) << 10) | ((a & 0x7fffffu) >> 13);
    const uint32_t rem = a & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

uint16_t fa_f32_to_bf16_bits(float x)
{
    uint32_t u = bits_of(x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

float fa_f16_bits_to_f32(uint16_t h)
{
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    if (e == 0x1fu) return float_of(sign | 0x7f800000u | (m << 13));
    if (e == 0) { const float v = (float)m * (1.0f / 16777216.0f); return sign ? -v : v; }
    return float_of(sign | ((e + 112u) << 23) | (m << 13));
}

float fa_bf16_bits_to_f32(uint16_t h) { return float_of((uint32_t)h << 16); }

static void normals4(uint64_t seed, uint32_t tensor, uint64_t group, float z[4])
{
    const uint32_t ctr[4] = {(uint32_t)group, (uint32_t)(group >> 32), tensor, 0u};
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t r[4];
    fa_philox4x32_10(ctr, key, r);
    const double two_pi = 6.283185307179586476925286766559;
    for (int pair = 0; pair < 2; ++pair) {
        const double u1 = ((double)r[2 * pair] + 0.5) * (1.0 / 4294967296.0);
        const double u2 = ((double)r[2 * pair + 1] + 0.5) * (1.0 / 4294967296.0);
        const double rad = sqrt(-2.0 * log(u1));
        z[2 * pair] = (float)(rad * cos(two_pi * u2));
        z[2 * pair + 1] = (float)(rad * sin(two_pi * u2));
    }
}

float fa_input_normal(uint64_t seed, uint32_t tensor, uint64_t index)
{
    float z[4];
    normals4(seed, tensor, index >> 2, z);
    return z[index & 3u];
}

int fa_input_row_selected(uint64_t seed, uint32_t tensor, uint64_t row, double fraction)
{
    if (!(fraction > 0.0)) return 0;
    const uint32_t ctr[4] = {(uint32_t)row, (uint32_t)(row >> 32), tensor, 1u};
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t r[4];
    fa_philox4x32_10(ctr, key, r);
    return (double)r[0] < fraction * 4294967296.0;
}

int fa_fill_normal(uint16_t *dst, uint64_t rows, int d, int dtype, uint64_t seed, uint32_t tensor,
                   float sigma, double fraction, float row_mult, int nthreads)
{
    if (!dst || d <= 0 || (d & 3) || (dtype != 0 && dtype != 1)) return -1;
    if (nthreads < 1) nthreads = 1;
#pragma omp parallel for num_threads(nthreads) schedule(static)
    for (int64_t row = 0; row < (int64_t)rows; ++row) {
        const float mult = fa_input_row_selected(seed, tensor, (uint64_t)row, fraction) ? sigma * row_mult : sigma;
        for (int t = 0; t < d; t += 4) {
            float z[4];
            const uint64_t index = (uint64_t)row * (uint64_t)d + (uint64_t)t;
            normals4(seed, tensor, index >> 2, z);
            for (int e = 0; e < 4; ++e) {
                const float x = z[e] * mult;
                dst[index + e] = dtype == 0 ? fa_f32_to_f16_bits(x) : fa_f32_to_bf16_bits(x);
            }
        }
    }
    return 0;
}
