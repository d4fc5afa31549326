// Where a walked 64-row tile of the backward kernels sits in LDS, as plain integer arithmetic shared by the
// device code and a host-side check (compiled as C by the tests): which 16-byte chunk of the source a direct
// global->LDS load instruction puts where, and which LDS byte each lane addresses in the two read patterns.
#ifndef FA_BWD_LAYOUT_H
#define FA_BWD_LAYOUT_H

#if defined(__HIPCC__)
#define FA_LAYOUT_HD __host__ __device__ __forceinline__
#else
#define FA_LAYOUT_HD static inline
#endif

// One 16-byte-chunk swizzle that serves both read patterns, so that the tile sits in LDS once.  A row holds
// cpr = D/8 chunks (16 at D = 128, 8 at D = 64); logical chunk c of row r is stored at chunk position c ^ swz(r).
// ds_read_b128 by 16 lanes on 16 consecutive rows and one logical chunk needs 16 different positions inside
// 256 bytes (a bijection of the row's low bits); ds_read_b64_tr_b16 by 32 lanes on 4 consecutive rows x 4
// consecutive chunks needs the 4 rows in 4 different 64-byte groups (the two high bits follow the row's low
// bits).  Invariant under row += 16, not under row += 8.
FA_LAYOUT_HD int fa_u_swz(int cpr, int row)
{
    return cpr == 16 ? (((row & 3) << 2) | ((row >> 2) & 3)) : ((((row >> 1) & 1) << 2) | ((row >> 2) & 3));
}

// Direct load: slot P (0 .. 64*cpr-1; lane l of the n-th wave instruction of a tile has P = 64 n + l) lands at LDS
// byte 16 P of the tile.  Returns the byte offset in the source tile it has to be fetched from.
FA_LAYOUT_HD int fa_bwd_load_source(int D, int P, int row_bytes)
{
    const int cpr = D / 8, row = P / cpr, pos = P % cpr;
    return row * row_bytes + ((pos ^ fa_u_swz(cpr, row)) << 4);
}

// ds_read_b128, A operand with rows = tile rows: lane (l32 = lane % 32, half = lane / 32) reads 16 bytes =
// head-dim values 16 s + 8 half .. + 7 of row l32 (+ 32 per row block, added as an immediate).
FA_LAYOUT_HD int fa_bwd_row_read(int D, int lane, int s)
{
    const int cpr = D / 8, half = lane >> 5, l32 = lane & 31;
    return l32 * D * 2 + (((2 * s + half) ^ fa_u_swz(cpr, l32)) << 4);
}

// ds_read_b64_tr_b16, A operand with rows = head dim (32-value block db), k = tile rows: the lane addresses the 8
// bytes = head-dim values 32 db + 16 (l32 / 16) + 4 (l16 % 4) .. + 3 of tile row 4 half + l16 / 4 + 8 hi (+ 16 per
// 16-row slice, added as an immediate); the instruction transposes among the 16 lanes that share l32 / 16 and half.
FA_LAYOUT_HD int fa_bwd_tr_read(int D, int lane, int db, int hi)
{
    const int cpr = D / 8, half = lane >> 5, l32 = lane & 31, l16 = lane & 15;
    const int row = 4 * half + (l16 >> 2) + 8 * hi, dq = l32 >> 4, c4 = l16 & 3;
    const int c = 4 * db + 2 * dq + (c4 >> 1);
    return row * D * 2 + ((c ^ fa_u_swz(cpr, row)) << 4) + ((c4 & 1) << 3);
}

// Where the 2 KiB dS block (32-query block qb, 32-key block kb) of a head lies in the five-product form's workspace,
// in blocks from the head's start.  Blocks are grouped in squares of 8 x 8 (256 queries x 256 keys, 128 KiB): the
// key-owning kernel (a workgroup = 8 key blocks, walking query tiles) and the query-owning kernel (a workgroup = 8
// query blocks, walking key tiles) then each work through one contiguous 128 KiB square for four tiles in a row
// (with whole block rows the query-owning kernel's eight waves read 512 KiB apart: 0.87 ms against 0.82 on B2 H32
// S8192 D128); inside a square the key block runs fastest, so the two blocks a query-owning wave needs per key tile
// are neighbours.
FA_LAYOUT_HD long long fa_ds_squares_per_side(int S) { return ((S + 31) / 32 + 7) / 8; }
FA_LAYOUT_HD long long fa_ds_blocks_per_head(int S) { return fa_ds_squares_per_side(S) * fa_ds_squares_per_side(S) * 64; }
FA_LAYOUT_HD long long fa_ds_block_index(int S, int qb, int kb)
{
    return (((long long)(qb >> 3) * fa_ds_squares_per_side(S) + (kb >> 3)) << 6) + ((qb & 7) << 3) + (kb & 7);
}

#endif
