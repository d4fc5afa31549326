// Kernel argument block of the gfx950 backward kernels (the reference has no backward pass).
#ifndef FA_BWD_ARGS_H
#define FA_BWD_ARGS_H
#include <stdint.h>

// One tensor [B, heads, rows, D] with a contiguous last dimension: element strides of the other three.
struct FaBwdTensor {
    long long bs, hs;
    int rs;
};

struct FaBwdArgs {
    const uint16_t *Q, *K, *V, *O, *dO;
    const float *lse;                       // [B,H,S] contiguous, natural log, as the forward pass writes it
    float *delta;                           // [B,H,S] scratch: sum_t dO*O per row, written by fa_bwd_dq
    float *lse2;                            // [B,H,S] scratch: lse * log2(e), +inf for rows that saw no key
    uint16_t *dQ, *dK, *dV;
    // Five-product form (reference layout only), or null: dS in blocks of 32 queries x 32 keys, 2 KiB each, block
    // (head bh, query block i, key block j) at (bh * fa_ds_blocks_per_head + fa_ds_block_index(i, j)) * 2 KiB
    // (fa_bwd_layout.h).  Inside a block the first KiB
    // holds, for 16-byte slot 32 h + k, key k against the queries 4 h + {0..3, 8..11}; the second KiB the same for
    // the queries 16 + 4 h + {0..3, 8..11} (h = 0, 1): the order in which fa_bwd_dkdv's lanes hold them.
    uint16_t *ds_blocks;
    const float *alibi;                     // [H] slopes or NULL
    FaBwdTensor q, k, v, o, dO_, dq, dk, dv;
    int B, H, Hk;                           // query heads, K/V heads (Hk divides H)
    // The K/V heads this launch works on, counted through the batch (batch * Hk + head): [head0, head0 + heads), and
    // with them the query heads [head0 * H/Hk, (head0 + heads) * H/Hk).  All of them, except in the five-product form
    // with a workspace that holds the dS blocks of only `ds_heads` K/V heads' groups at a time: then the key-owning
    // and the query-owning kernel are launched once per such chunk, and block addresses count from the chunk's start.
    int head0, heads, ds_heads;
    int S, Sk;                              // queries, keys; query i sits at key position i + Sk - S
    int L, R;                               // key j visible to the query at position p iff p - L <= j <= p + R
    float scale;
    unsigned drop_threshold;                // dropout: keep iff the key's byte >= threshold (p in units of 1/256); 0 = none
    float drop_scale;                       // 256 / (256 - threshold)
    unsigned seed_lo, seed_hi;
};

#endif
