// Kernel argument block of the gfx950 forward kernel.
// Plays the part of the reference's mykernelParamType (reference
// include/utils.h:143-165) on the device side: pointers, sizes, the folded
// softmax scale and the effective mask bounds.
#ifndef FA_KERNEL_ARGS_H
#define FA_KERNEL_ARGS_H
#include <stdint.h>

struct FaKernelArgs {
    const uint16_t *Q;
    const uint16_t *K;
    const uint16_t *V;
    uint16_t *O;
    float *lse;          // may be null
    const float *alibi;  // per-head ALiBi slopes [H], or null
    int H;               // heads per batch entry
    int BH;              // batch * heads
    int S;
    int n_qblocks;       // query blocks per head
    int descending;      // 1: item rank 0 is the last query block (longest first)
    int L;               // key j visible to query i iff i - L <= j <= i + R
    int R;
    float scale;         // softmax scale
    float scale_log2e;   // softmax scale * log2(e)
    long long n_items;   // work items: BH * n_qblocks
    unsigned *queue;     // null, or 9 counters of a work queue: next list position per XCD [0..7], finished workgroups [8]
    // --- used by the GENERAL and STRIDED instantiations only (strides in elements; the head dimension is contiguous)
    int Hk;              // K/V heads per batch entry; query head h reads K/V head h / (H / Hk)
    int q_rs, k_rs, v_rs, o_rs;                 // row (sequence position) strides
    long long q_bs, q_hs, k_bs, k_hs;           // batch and head strides
    long long v_bs, v_hs, o_bs, o_hs;
    int Sk;              // keys per head (S is the number of queries); query i sits at key position i + Sk - S
    int n_splits;        // > 1: every (head, query block) is n_splits consecutive work items, each over
    int tiles_per_split; //      tiles_per_split key tiles, writing partial results:
    float *o_part;       //      [n_splits][BH][S][D] fp32, normalised over the split's own keys
    float *lse_part;     //      [n_splits][BH][S] fp32, -inf where the split saw no key of the row
    int pack;            // > 1: work items are (batch, K/V head) and their rows the queries of the `pack` query
                         //      heads of that K/V head, head after head (n_qblocks is 1)
    // --- used by the DROPOUT instantiations only
    unsigned drop_threshold;   // key kept iff its byte >= threshold; p = threshold / 256
    float drop_scale;          // 256 / (256 - threshold)
    unsigned seed_lo, seed_hi;
    // --- masked instantiations
    int exact_first_rows;      // 1: no row is recomputed in the reference verifier's rounded-product arithmetic
#ifdef FA_CHECK_RING
    // checking build only: [0] comparisons made, [1] LDS bytes that were not the tile the iteration expected
    unsigned long long *ring_check;
#endif
};

#endif
