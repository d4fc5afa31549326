/*
 * Backward pass of the MI355X (gfx950) FlashAttention library: dQ, dK, dV from Q, K, V, O, dO and the
 * logsumexp that fa_fwd() / run_flash_attention() write to L.
 *
 * No counterpart in the reference: its operator is forward only and its L argument is accepted and never
 * written (reference src/flash_forward.h:602,628-644).  This is the consumer of the logsumexp this library
 * adds.  Same C ABI conventions as fa_fwd.h: plain pointers and ints, an int status, nothing is allocated.
 *
 * Supported: the reference's layout only, contiguous [B,N,S,d] fp16 or bf16 with S a multiple of 128 and d 64
 * or 128; causal and one- or two-sided window masks.  Not in the parameter block, hence not supported: ALiBi, dropout, strides, grouped K/V heads;
 * other lengths are refused with FA_ERR_SEQLEN_MULTIPLE.
 */
#ifndef FA_BWD_H
#define FA_BWD_H
#include "fa_fwd.h"
#ifdef __cplusplus
extern "C" {
#endif

typedef struct fa_bwd_params {
    const void *Q, *K, *V;    /* [B,N,S,d] device, the forward inputs                                  */
    const void *O;            /* [B,N,S,d] device, the forward output                                  */
    const void *dO;           /* [B,N,S,d] device, gradient of the loss with respect to O              */
    const float *L;           /* [B,N,S] fp32 logsumexp written by the forward pass                     */
    void *dQ, *dK, *dV;       /* [B,N,S,d] device, fully overwritten, same type as the inputs           */
    int B, N, S, d;
    float softmax_scale;
    int window_size_left;     /* as in fa_fwd_params                                                   */
    int window_size_right;
    int dtype;                /* FA_DTYPE_F16 / FA_DTYPE_BF16                                          */
    int is_causal;
    void *workspace;          /* device scratch, at least fa_bwd_workspace_bytes(): B*N*S floats         */
    unsigned long long workspace_bytes;
} fa_bwd_params;

int fa_bwd_validate(const fa_bwd_params *p);
unsigned long long fa_bwd_workspace_bytes(const fa_bwd_params *p);
/* Enqueues two kernels on `stream` (dQ and the row sums of dO*O, then dK and dV) and returns without
 * synchronising.  No atomics: the same inputs give the same bits on every run. */
int fa_bwd(const fa_bwd_params *p, void *stream);
/* Algorithmic FLOPs of the backward pass: 10 * B * N * d * pairs (five products over the unmasked pairs). */
double fa_bwd_algorithmic_flops(int B, int N, int S, int d, int is_causal, int window_left, int window_right);

#ifdef __cplusplus
}
#endif
#endif
