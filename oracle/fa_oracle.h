/*
 * CPU oracle for the FlashAttention forward path: TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the reference's CPU verifier
 * (reference src/main.cu:159-268, attention_forward_cpu) with the same
 * rounding points, extended with a logsumexp output, a bf16 storage mode,
 * one-sided windows, row-subset evaluation and an unrounded fp64 mode.
 * Nothing in the product library links or calls this; only the test-suite,
 * the smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Pinning status (what checks this restatement against something other than
 * itself): the reference holds no golden vectors for this path, so the
 * oracle is pinned by closed forms, invariants, brute-force fp64 fixtures and
 * torch's scaled_dot_product_attention in tests/test_oracle.py, and every
 * rounding point of main.cu:193,259,261 (half product, p rounded to half,
 * half product with v) by bit equality with an independent literal written in
 * numpy float16 / torch bfloat16 arithmetic in the same file.  Bit-exact
 * agreement with the CUDA host `__half` operators of the reference build is
 * "parity unpinned": it follows from source semantics (float multiply of two
 * halves is exact, then one round-to-nearest-even) but no reference binary
 * can be run here.  Dropout is also "parity unpinned" against the reference,
 * by construction: the reference's kernel draws from per-thread curand states
 * and its verifier skips dropout runs (main.cu:102); the decision function
 * used here is a counter-based replacement, pinned by the Random123 known
 * answers, a numpy implementation and a mask read-back in the same tests.
 */
#ifndef FA_ORACLE_H
#define FA_ORACLE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

enum { FA_ORACLE_F16 = 0, FA_ORACLE_BF16 = 1 };

typedef struct fa_oracle_cfg {
    int B, H, S, D;        /* tensors are contiguous [B,H,S,D]; main.cu:182 */
    int dtype;             /* FA_ORACLE_F16 / FA_ORACLE_BF16 storage type     */
    float scale;           /* softmax scale, main.cu:163,195                  */
    int causal;            /* j > i masked, main.cu:210-218                   */
    int window_left;       /* i - j > window_left masked  when >= 0           */
    int window_right;      /* j - i > window_right masked when >= 0           */
                           /* reference window_size w (main.cu:220-229) is
                              window_left = window_right = w                  */
    const float *alibi_slopes; /* [H] or NULL, main.cu:200-207                */
    /* Dropout (GPU side of the reference only, flash_forward.h:248-265; its CPU verifier skips dropout runs,
       main.cu:102): every normalised probability is zeroed when its random byte is below the threshold and
       multiplied by 256/(256-threshold) otherwise, before it is rounded to the storage type; the logsumexp is
       untouched.  threshold 0 = no dropout. */
    int dropout_threshold;     /* 0..255: drop probability in units of 1/256  */
    uint64_t dropout_seed;
} fa_oracle_cfg;

/* The dropout decision for (bh = b*H + h, query i, key j): 1 = kept.  Byte 4*((j%32)/8) + j%4 of the
 * Philox4x32-10 block with counter (2*(j/32) + (j/4)%2, i, bh, 0x44524F50) and key (seed low, seed high),
 * compared with the threshold. */
int fa_oracle_dropout_keep(uint64_t seed, int64_t bh, int i, int j, int threshold);
/* Philox4x32-10 as published (Salmon et al., Random123), exposed for its known-answer tests. */
void fa_oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);

/* Scalar conversions (round-to-nearest-even), exposed for the tests. */
uint16_t fa_oracle_f32_to_f16(float x);
float    fa_oracle_f16_to_f32(uint16_t h);
uint16_t fa_oracle_f32_to_bf16(float x);
float    fa_oracle_bf16_to_f32(uint16_t h);

/*
 * Faithful evaluation of selected rows.  rows[n] is a flat row index
 * (b*H + h)*S + i.  O_rows is [nrows, D] in the storage dtype, lse_rows is
 * [nrows] fp32 (natural log; max + logf(sum) of the scaled, masked scores).
 * Either output may be NULL.  Returns 0, or -1 on bad arguments.
 */
int fa_oracle_rows(const fa_oracle_cfg *cfg, const uint16_t *Q, const uint16_t *K,
                   const uint16_t *V, const int64_t *rows, int64_t nrows,
                   uint16_t *O_rows, float *lse_rows, int nthreads);

/* Whole tensor: O is [B,H,S,D], lse is [B,H,S]. */
int fa_oracle_full(const fa_oracle_cfg *cfg, const uint16_t *Q, const uint16_t *K,
                   const uint16_t *V, uint16_t *O, float *lse, int nthreads);

/* Same rows with no intermediate rounding at all: inputs widened to double,
 * everything accumulated in double.  Used to measure how much of the
 * tolerance the faithful path's own half-precision products consume. */
int fa_oracle_rows_f64(const fa_oracle_cfg *cfg, const uint16_t *Q, const uint16_t *K,
                       const uint16_t *V, const int64_t *rows, int64_t nrows,
                       double *O_rows, double *lse_rows, int nthreads);

/* The literal reference algorithm with its S*S score buffer and its loop
 * order (main.cu:176-266), single-threaded, small shapes only.  Exists so the
 * streamed row evaluation above can be checked bit-for-bit against the
 * reference's own structure. */
int fa_oracle_literal(const fa_oracle_cfg *cfg, const uint16_t *Q, const uint16_t *K,
                      const uint16_t *V, uint16_t *O);

/*
 * Gradients of sum(dO * O) with respect to Q, K, V in fp64: dQ, dK, dV are [B,H,S,D] doubles.  The reference has
 * no backward pass; this is the textbook derivative (dV = P^T dO, dP = dO V^T, dS = P o (dP - rowsum(dO o O)),
 * dQ = scale dS K, dK = scale dS^T Q) on the storage-type inputs, with the same masks and ALiBi bias as the
 * forward functions and dropout decisions (O = sum_j m_ij p_ij v_j with m_ij = keep_ij / (1 - p): m scales dV's P and
 * dP, the softmax Jacobian sees the undropped p).
 */
int fa_oracle_bwd_f64(const fa_oracle_cfg *cfg, const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                      const uint16_t *dO, double *dQ, double *dK, double *dV, int nthreads);

#ifdef __cplusplus
}
#endif
#endif
