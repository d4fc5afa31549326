/* Host-side check of the LDS layout arithmetic the backward kernels share with this file
 * (flash-attn-rtx5060_amd/csrc/fa_bwd_layout.h).  Exit status 0 = all properties hold.
 *  1. what the direct loads put into LDS is what the two read patterns expect to find at the bytes they address;
 *  2. all addresses stay inside the 64-row tile;
 *  3. neither read pattern has an LDS bank conflict: the 16 lanes of one ds_read_b128 pass cover 16 different
 *     16-byte positions of a 256-byte bank row, the 32 lanes of one ds_read_b64_tr_b16 pass 32 different 8-byte
 *     positions. */
#include <stdio.h>
#include <string.h>
#include "fa_bwd_layout.h"

static int fails = 0;
#define CHECK(cond, ...) do { if (!(cond)) { if (fails++ < 20) { printf(__VA_ARGS__); printf("\n"); } } } while (0)

static void check(int D)
{
    const int cpr = D / 8, rowb = D * 2, tileb = 64 * rowb;
    /* lds_row[chunk position], lds_chunk[...]: which source (row, logical chunk) each 16-byte LDS slot holds */
    static int lds_row[64 * 16], lds_chunk[64 * 16];
    static int seen[64 * 16];
    memset(seen, 0, sizeof(seen));
    for (int P = 0; P < 64 * cpr; ++P) {
        const int src = fa_bwd_load_source(D, P, rowb);          /* contiguous source tile */
        CHECK(src >= 0 && src + 16 <= tileb && src % 16 == 0, "D=%d P=%d: source offset %d outside the tile", D, P, src);
        lds_row[P] = src / rowb;
        lds_chunk[P] = (src % rowb) / 16;
        CHECK(lds_row[P] == P / cpr, "D=%d P=%d: a slot of LDS row %d is filled from source row %d", D, P, P / cpr, lds_row[P]);
        seen[lds_row[P] * cpr + lds_chunk[P]]++;
    }
    for (int i = 0; i < 64 * cpr; ++i) CHECK(seen[i] == 1, "D=%d: source chunk %d loaded %d times", D, i, seen[i]);
    /* with a row stride the source offset moves by row * (stride - rowb) and nothing else */
    for (int P = 0; P < 64 * cpr; ++P)
        CHECK(fa_bwd_load_source(D, P, 3 * rowb + 16) - fa_bwd_load_source(D, P, rowb) == (P / cpr) * (2 * rowb + 16),
              "D=%d P=%d: row stride handled wrongly", D, P);

    /* row-wise reads: lane (l32, half), slice s, row block b -> row 32 b + l32, head-dim chunk 2 s + half */
    for (int b = 0; b < 2; ++b)
        for (int s = 0; s < D / 16; ++s) {
            int pos_used[4][16];
            memset(pos_used, 0, sizeof(pos_used));
            for (int lane = 0; lane < 64; ++lane) {
                const int addr = fa_bwd_row_read(D, lane, s) + b * 32 * rowb;
                CHECK(addr >= 0 && addr + 16 <= tileb && addr % 16 == 0, "D=%d row read out of the tile: lane %d s %d b %d", D, lane, s, b);
                const int slot = addr / 16;
                CHECK(lds_row[slot] == 32 * b + (lane & 31) && lds_chunk[slot] == 2 * s + (lane >> 5),
                      "D=%d row read: lane %d s %d b %d finds row %d chunk %d", D, lane, s, b, lds_row[slot], lds_chunk[slot]);
                pos_used[lane / 16][(addr / 16) % 16]++;
            }
            for (int pass = 0; pass < 4; ++pass)
                for (int q = 0; q < 16; ++q) CHECK(pos_used[pass][q] == 1, "D=%d row read: bank conflict, s %d b %d pass %d", D, s, b, pass);
        }

    /* transposed reads: lane -> 8 bytes = head-dim values 32 db + 16 (l32/16) + 4 (l16%4) .. +3 of tile row
       16 t2 + 8 hi + 4 half + l16/4 */
    for (int t2 = 0; t2 < 4; ++t2)
        for (int db = 0; db < D / 32; ++db)
            for (int hi = 0; hi < 2; ++hi) {
                int pos_used[2][32];
                memset(pos_used, 0, sizeof(pos_used));
                for (int lane = 0; lane < 64; ++lane) {
                    const int half = lane >> 5, l32 = lane & 31, l16 = lane & 15;
                    const int addr = fa_bwd_tr_read(D, lane, db, hi) + 16 * t2 * rowb;
                    CHECK(addr >= 0 && addr + 8 <= tileb && addr % 8 == 0, "D=%d transposed read out of the tile: lane %d", D, lane);
                    const int slot = addr / 16, want_row = 16 * t2 + 8 * hi + 4 * half + (l16 >> 2);
                    const int want_value = 32 * db + 16 * (l32 >> 4) + 4 * (l16 & 3);          /* first of 4 head-dim values */
                    CHECK(lds_row[slot] == want_row && lds_chunk[slot] * 8 + (addr % 16) / 2 == want_value,
                          "D=%d transposed read: lane %d t2 %d db %d hi %d finds row %d value %d, wants row %d value %d", D, lane, t2, db, hi,
                          lds_row[slot], lds_chunk[slot] * 8 + (addr % 16) / 2, want_row, want_value);
                    pos_used[half][(addr / 8) % 32]++;
                }
                for (int pass = 0; pass < 2; ++pass)
                    for (int q = 0; q < 32; ++q) CHECK(pos_used[pass][q] == 1, "D=%d transposed read: bank conflict, t2 %d db %d hi %d", D, t2, db, hi);
            }
}

int main(void)
{
    check(64);
    check(128);
    printf("%s (%d failed checks)\n", fails ? "FAILED" : "ok", fails);
    return fails ? 1 : 0;
}
