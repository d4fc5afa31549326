// Kernel argument block of the gfx950 backward kernels (the reference has no backward pass).
#ifndef FA_BWD_ARGS_H
#define FA_BWD_ARGS_H
#include <stdint.h>

struct FaBwdArgs {
    const uint16_t *Q, *K, *V, *O, *dO;     // contiguous [B,H,S,D]
    const float *lse;                       // [B,H,S], natural log, as the forward pass writes it
    float *delta;                           // [B,H,S] scratch: sum_t dO*O per row
    uint16_t *dQ, *dK, *dV;                 // contiguous [B,H,S,D]
    int BH, S;
    int L, R;                               // key j visible to query i iff i - L <= j <= i + R
    float scale;
};

#endif
