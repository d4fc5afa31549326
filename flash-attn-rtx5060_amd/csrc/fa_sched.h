// Tile scheduler arithmetic shared by the gfx950 kernel and its host mirror.
//
// Replaces the reference's in-kernel Schedule<0,...>::next
// (reference src/flash_forward.h:43-64): the same key-tile clipping for causal
// and local masks, but with one-sided windows, a longest-first work order and
// a per-tile classification so that element masks are applied only where a
// tile straddles a mask edge and fully masked tiles are never visited
// (the reference masks every tile, src/mask.h:10-84).
#ifndef FA_SCHED_H
#define FA_SCHED_H

#if defined(__HIPCC__)
#define FA_HD __host__ __device__ __forceinline__
#else
#define FA_HD static inline
#endif

// Effective mask bounds: key j is visible to query i iff  i - L <= j <= i + R.
// `S` stands in for "unbounded" (no |i-j| can reach it).
FA_HD void fa_mask_bounds(int S, int is_causal, int window_left, int window_right, int *L, int *R)
{
    int r = (window_right < 0 || window_right > S) ? S : window_right;
    int l = (window_left < 0 || window_left > S) ? S : window_left;
    if (is_causal) r = 0;
    *L = l;
    *R = r;
}

// Inclusive key-tile range visited by query rows [q_begin, q_begin + rows).
FA_HD void fa_tile_range(int S, int block_keys, int L, int R, int q_begin, int rows, int *tile_lo, int *tile_hi)
{
    int lo_key = q_begin - L;
    if (lo_key < 0) lo_key = 0;
    int hi_key = q_begin + rows - 1 + R;
    if (hi_key > S - 1) hi_key = S - 1;
    if (hi_key < lo_key) {      // no visible key at all (queries placed before the first key, or past the last)
        *tile_lo = 1;
        *tile_hi = 0;
        return;
    }
    *tile_lo = lo_key / block_keys;
    *tile_hi = hi_key / block_keys;
}

// 0 = every (query,key) pair masked, 2 = none masked, 1 = mixed.
FA_HD int fa_tile_class(int block_keys, int L, int R, int q_begin, int rows, int tile)
{
    const int k0 = tile * block_keys, k1 = k0 + block_keys - 1;
    const int qa = q_begin, qb = q_begin + rows - 1;
    if (k0 > qb + R || k1 < qa - L) return 0;
    if (k1 <= qa + R && k0 >= qb - L) return 2;
    return 1;
}

// Work item `item` (0 is dispatched first) -> (batch*heads + head, query block).
//
// Heads are taken in groups of FA_HEAD_GROUP = 8, one head per XCD: the hardware deals consecutively
// dispatched workgroups round-robin over the eight XCDs, so with the head index fastest inside a group,
// head (8g + x) runs on XCD x only, and the whole chip works on eight heads at a time.  One head's K and V
// (4 MiB at seqlen 8192, head dim 128) then fit that XCD's L2 and are fetched from HBM about once instead of
// once per query block.  Inside a group the query blocks are ordered by decreasing number of key tiles
// (longest first): with a causal or left-window mask the tile count grows with the query block index, so
// the last query block of every head goes first and the short ones fill the tail.
#define FA_HEAD_GROUP 8
FA_HD void fa_item_decode(long long item, int BH, int n_qblocks, int descending, int *bh, int *qblock)
{
    // (list positions and FA_HEAD_GROUP * n_qblocks fit 31 bits, which the host checks before a launch: 32-bit
    // unsigned divisions, a few instructions each on the GPU where a 64-bit one is a long subroutine that every
    // work item would pay for three times)
    const unsigned it = (unsigned)item;
    const unsigned per_group = (unsigned)FA_HEAD_GROUP * (unsigned)n_qblocks;
    const unsigned full_groups = (unsigned)BH / FA_HEAD_GROUP;
    unsigned group = it / per_group;
    unsigned heads_here = FA_HEAD_GROUP;
    if (group >= full_groups) {          // the last, smaller group
        group = full_groups;
        heads_here = (unsigned)BH - full_groups * FA_HEAD_GROUP;
    }
    const unsigned rem = it - group * per_group;
    const unsigned rank = rem / heads_here;
    *bh = (int)(group * FA_HEAD_GROUP + (rem - rank * heads_here));
    *qblock = descending ? (n_qblocks - 1 - (int)rank) : (int)rank;
}

// List head index `bh` (batch * heads + position in the batch entry's list) -> batch entry, query head and K/V
// head of a work item of the regular problem with grouped K/V heads.  With as many K/V heads as query heads the
// list position is the head; with groups of H / Hk query heads per K/V head, position r stands for K/V head
// r % Hk and the (r / Hk)-th query head of its group: the list walks the K/V heads fastest, so that with the
// head index dealt round robin over the XCDs (fa_item_decode) the query heads of one K/V head run on the XCD
// whose L2 holds its K and V.  (32-bit unsigned divisions; all operands are uniform.)
FA_HD int fa_strided_heads(int bh, int H, int Hk, int *hi, int *hk)
{
    const unsigned bi = (unsigned)bh / (unsigned)H, r = (unsigned)bh - bi * (unsigned)H;
    unsigned q = r, k = r;
    if (Hk != H) {
        const unsigned member = r / (unsigned)Hk;
        k = r - member * (unsigned)Hk;
        q = k * ((unsigned)H / (unsigned)Hk) + member;
    }
    *hi = (int)q;
    *hk = (int)k;
    return (int)bi;
}

#endif
