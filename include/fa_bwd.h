/*
 * Backward pass of the MI355X (gfx950) FlashAttention library: dQ, dK, dV from Q, K, V, O, dO and the
 * logsumexp that fa_fwd() / run_flash_attention() write to L.
 *
 * No counterpart in the reference: its operator is forward only and its L argument is accepted and never
 * written (reference src/flash_forward.h:602,628-644).  This is the consumer of the logsumexp this library
 * adds.  Same C ABI conventions as fa_fwd.h: plain pointers and ints, an int status, nothing is allocated.
 *
 * Layouts as in fa_fwd(): fp16 or bf16, d 64 or 128, any S >= 1, contiguous [B,N,S,d] or element strides with a
 * contiguous last dimension, K/V with n_kv_heads heads (dK and dV are summed over the query heads of a group) and
 * S_kv keys (query i sits at key position i + S_kv - S), causal and one- or two-sided window masks, ALiBi,
 * dropout (the forward's decisions are replayed from its seed, nothing is stored).  Key splits do not apply.
 */
#ifndef FA_BWD_H
#define FA_BWD_H
#include "fa_fwd.h"
#ifdef __cplusplus
extern "C" {
#endif

typedef struct fa_bwd_params {
    const void *Q, *K, *V;    /* device, the forward inputs: Q [B,N,S,d]; K, V [B,n_kv_heads,S_kv,d]              */
    const void *O;            /* [B,N,S,d] device, the forward output                                          */
    const void *dO;           /* [B,N,S,d] device, gradient of the loss with respect to O                      */
    const float *L;           /* [B,N,S] contiguous fp32 logsumexp written by the forward pass.  Run that pass
                                 with fa_fwd_params.exact_first_rows = 1: the backward pass recomputes P from
                                 exact scores, and the default forward writes the first 32 rows of a causal
                                 head (rows that see at most 32 keys) in the reference verifier's
                                 rounded-product arithmetic.  With the default forward's O and L those rows'
                                 gradients are still within 2e-3 (fp16) / 1.6e-2 (bf16) of the largest
                                 gradient at unit-variance inputs (tests/test_gpu_parity_bwd.py); every other
                                 row is unaffected                                                             */
    void *dQ, *dK, *dV;       /* device, shaped like Q, K, V; fully overwritten, same type as the inputs        */
    int B, N, S, d;
    float softmax_scale;
    int window_size_left;     /* as in fa_fwd_params                                                           */
    int window_size_right;
    int dtype;                /* FA_DTYPE_F16 / FA_DTYPE_BF16                                                  */
    int is_causal;
    void *workspace;          /* device scratch, at least fa_bwd_workspace_bytes(): 2*B*N*S floats; with at least
                                 fa_bwd_fast_workspace_bytes() (when that is not 0) the five-product form runs   */
    unsigned long long workspace_bytes;
    /* ---- general layouts; all zero = the reference's contiguous [B,N,S,d] with S_kv = S ---- */
    int n_kv_heads;           /* 0 = N; otherwise divides N                                                    */
    int S_kv;                 /* 0 = S                                                                         */
    const float *alibi_slopes_ptr;   /* [N] fp32 device or NULL, as in fa_fwd_params                            */
    long long q_strides[3];   /* element strides of (batch, head, row); {0,0,0} = contiguous                   */
    long long k_strides[3];
    long long v_strides[3];
    long long o_strides[3];
    long long do_strides[3];
    long long dq_strides[3];
    long long dk_strides[3];
    long long dv_strides[3];
    float dropout_prob;       /* the forward's; 0 = none.  The keep decisions are replayed from (seed, head, query, key) */
    unsigned long long seed;  /* the forward's                                                                  */
} fa_bwd_params;

int fa_bwd_validate(const fa_bwd_params *p);
unsigned long long fa_bwd_workspace_bytes(const fa_bwd_params *p);
/* The workspace size that selects the five-product form, or 0 when the problem has none (it needs as many
 * keys as queries; any storage order and grouping of K/V heads; dropout or ALiBi, not both, and only when S is a
 * multiple of 128): the small
 * workspace plus B*N*S*S storage-type elements (B2 N32 S8192: 8.6 GB).  With it, the key-owning kernel writes every
 * dS block it forms and dQ is one product over those blocks, instead of a second recomputation of S and dP. */
unsigned long long fa_bwd_fast_workspace_bytes(const fa_bwd_params *p);
/* The five-product form also runs with less: the dS blocks of as many K/V heads (with their groups of query heads)
 * at a time as the workspace holds, a multiple of eight, the two kernels launched once per such chunk; same bits as
 * with the full size.  This is the smallest workspace that selects it (0 when fa_bwd_fast_workspace_bytes is 0):
 * the small workspace plus the blocks of enough heads for two rounds of key blocks over the chip (B2 N32 S8192:
 * 16 heads, 2.1 GB).  Anything below it selects the seven-product form. */
unsigned long long fa_bwd_min_fast_workspace_bytes(const fa_bwd_params *p);
/* Enqueues the backward pass on `stream` and returns without synchronising: two kernels (dQ and the row sums of
 * dO*O, then dK and dV: seven matrix products), or, with the large workspace, three (the row sums; dK, dV and the
 * dS blocks; dQ from the blocks: five products).  No atomics either way: every output element has one writer and
 * the same inputs give the same bits on every run. */
int fa_bwd(const fa_bwd_params *p, void *stream);
/* Host mirror of the arithmetic with which the key-owning kernel finds its work (csrc/fa_sched.h with the two
 * sides of the mask exchanged and shifted by S_kv - S): the inclusive range of 64-query tiles that contain a
 * query seeing at least one of the keys [k_begin, k_begin + rows), lo > hi when there is none; and the class of
 * one such tile (0 = no pair visible, 2 = all visible, 1 = mixed).  S_kv = 0 means S. */
void fa_bwd_sched_query_tile_range(int S, int S_kv, int is_causal, int window_left, int window_right,
                                   int k_begin, int rows, int *tile_lo, int *tile_hi);
int fa_bwd_sched_classify(int S, int S_kv, int is_causal, int window_left, int window_right,
                          int k_begin, int rows, int tile);
/* Algorithmic FLOPs of the backward pass: 10 * B * N * d * pairs (five products over the unmasked pairs). */
double fa_bwd_algorithmic_flops(int B, int N, int S, int d, int is_causal, int window_left, int window_right);

#ifdef __cplusplus
}
#endif
#endif
