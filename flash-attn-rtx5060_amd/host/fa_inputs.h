/*
 * Seeded counter-based input generator of the host harness.
 *
 * Takes the place of the reference's input initialisation
 * (reference src/main.cu:69-81: std::default_random_engine(26), U(0,10),
 * interleaved Q,K,V draws) and of the slot its curand state initialiser
 * occupies (reference src/init_curand_states.h:7-14).  Every element is a pure
 * function of (seed, tensor id, flat [B,N,S,d] index): Philox4x32-10 keyed by
 * the seed, counter = (index / 4, tensor id, stream), Box-Muller in double,
 * one rounding to fp32, scaling, one round-to-nearest-even to the storage
 * type.  The same host buffer is copied to the GPU and handed to the CPU
 * verifier, so both see identical inputs by construction.
 */
#ifndef FA_INPUTS_H
#define FA_INPUTS_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum { FA_TENSOR_Q = 0, FA_TENSOR_K = 1, FA_TENSOR_V = 2 };

/* Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11). */
void fa_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);

uint16_t fa_f32_to_f16_bits(float x);
uint16_t fa_f32_to_bf16_bits(float x);
float fa_f16_bits_to_f32(uint16_t h);
float fa_bf16_bits_to_f32(uint16_t h);

/* The fp32 normal deviate of element `index` of tensor `tensor`, before scaling. */
float fa_input_normal(uint64_t seed, uint32_t tensor, uint64_t index);
/* 1 if row `row` (flat (b*N+h)*S+i) of tensor `tensor` is one of the seeded
 * `fraction` of rows that get multiplied by `row_mult`. */
int fa_input_row_selected(uint64_t seed, uint32_t tensor, uint64_t row, double fraction);

/*
 * dst[n] = storage(sigma * z(seed,tensor,n) * (row selected ? row_mult : 1)),
 * n in [0, rows*d).  dtype: 0 = fp16, 1 = bf16.  fraction == 0 disables the
 * row scaling.  Returns 0, -1 on bad arguments.
 */
int fa_fill_normal(uint16_t *dst, uint64_t rows, int d, int dtype, uint64_t seed, uint32_t tensor,
                   float sigma, double fraction, float row_mult, int nthreads);

#ifdef __cplusplus
}
#endif
#endif
