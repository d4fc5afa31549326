// FlashAttention forward for gfx950 (MI355X), hand-written HIP.
//
// Role of the reference's forward_kernel<> (reference src/flash_forward.h:78-366)
// with its helpers apply_softmax (src/softmax.h:9-86) and apply_mask
// (src/mask.h:10-84), designed for CDNA4 instead of translated:
//
//  * Transposed formulation.  Each wave owns 32 query rows and computes
//    S^T = K * Q^T with v_mfma_f32_32x32x16 (M = keys, N = queries), so a lane
//    holds ONE query column and 16 key rows of every 32x32 block.  The online
//    softmax reductions (softmax.h:19-41,69-78 use quad shuffles) are then
//    in-register plus one v_permlane32_swap between the two half-waves.
//  * The S^T accumulator layout is exactly the B-operand layout of the second
//    contraction O^T = V^T * P^T, so P never leaves registers (the role of the
//    C->A fragment repack at flash_forward.h:269-278).  O^T keeps the query on
//    the lane as well, so the rescale factor is a per-lane scalar.
//  * V^T operands come from row-major V tiles in LDS through
//    ds_read_b64_tr_b16 (the role of ldmatrix.trans, include/utils.h:38-45).
//  * K/V tiles are XOR-swizzled at 16-byte granularity so that both the
//    ds_read_b128 K-operand pattern and the transposed V pattern are free of
//    bank conflicts without padding (the reference tiles are unswizzled,
//    utils.h:168).
//  * exp2 with scale*log2(e) folded into one FMA, the rescale of O done only
//    when a row maximum has grown by more than 2^8 (the reference recomputes
//    the factor 4*d/8 times per tile, flash_forward.h:296-299), the -inf
//    guard the reference lacks (softmax.h:55,83).
//  * Masks are evaluated per element only on tiles that straddle a mask edge,
//    and tiles that are fully masked for a wave are skipped by that wave.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include "fa_kernel_args.h"
#include "fa_sched.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kBlockKeys = 64;          // keys per K/V tile
constexpr float kRescaleLog2 = 8.0f;    // rescale O only when a row max grew by > 2^8

template <bool BF16> struct Num;
template <> struct Num<false> {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    }
    static __device__ __forceinline__ float add_pair(uint32_t p, float acc)
    {
        const f16x2 one = {(_Float16)1.0f, (_Float16)1.0f};
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, p), one, acc, false);
    }
};
template <> struct Num<true> {
    static __device__ __forceinline__ f32x16 mfma(u32x4 a, u32x4 b, f32x16 c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi)
    {
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    static __device__ __forceinline__ float add_pair(uint32_t p, float acc)
    {
        const bf16x2 one = {(__bf16)1.0f, (__bf16)1.0f};
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, p), one, acc, false);
    }
};

// 16-byte-chunk swizzles.  A tile row holds CPR = D/8 chunks.
// K is read with ds_read_b128 by 16 lanes holding 16 consecutive rows and one
// logical chunk: those must land on 16 different 16-byte bank groups.
template <int CPR> __device__ __forceinline__ int k_swz(int row) { return CPR == 16 ? (row & 15) : ((row >> 1) & 7); }
// V is read with ds_read_b64_tr_b16: 32 lanes cover 4 consecutive rows x 4
// consecutive chunks; the 4 rows must land on 4 different 64-byte bank groups.
template <int CPR> __device__ __forceinline__ int v_swz(int row) { return CPR == 16 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); }

__device__ __forceinline__ float swap_halves(float x)
{
    // lane l <-> lane l^32
    auto r = __builtin_amdgcn_permlane32_swap(__builtin_bit_cast(uint32_t, x), __builtin_bit_cast(uint32_t, x), false, false);
    return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}

__device__ __forceinline__ u32x4 lds_read_b128(uint32_t addr)
{
    return *(const __attribute__((address_space(3))) u32x4 *)addr;
}
__device__ __forceinline__ u32x2 lds_read_tr(uint32_t addr)
{
    i16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4 *)addr);
    return __builtin_bit_cast(u32x2, v);
}
__device__ __forceinline__ void lds_write_b128(uint32_t addr, u32x4 v)
{
    *(__attribute__((address_space(3))) u32x4 *)addr = v;
}

template <bool BF16, int D, int NW, bool MASKED>
__global__ void __launch_bounds__(NW * 64) fa_fwd_kernel(const FaKernelArgs a)
{
    constexpr int BR = 32 * NW;
    constexpr int NT = 64 * NW;
    constexpr int CPR = D / 8;                    // 16-byte chunks per row
    constexpr int ROWB = D * 2;                   // bytes per row
    constexpr int TILEB = kBlockKeys * ROWB;      // bytes per K (or V) tile
    constexpr int CHUNKS = kBlockKeys * CPR;      // chunks per tile
    constexpr int LPT = CHUNKS / NT;              // chunks per thread per tensor
    constexpr int KS = D / 16;                    // k-slices of the QK contraction
    constexpr int DB = D / 32;                    // 32-wide blocks of head dim
    static_assert(CHUNKS % NT == 0, "tile must divide over the workgroup");
    typedef Num<BF16> N;

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;   // stage s: K at s*2*TILEB, V at s*2*TILEB + TILEB

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int half = lane >> 5, l32 = lane & 31, l16 = lane & 15;

    int bh, qblock;
    fa_item_decode((long long)blockIdx.x, a.BH, a.n_qblocks, a.descending, &bh, &qblock);
    const int S = a.S;
    const size_t head_off = (size_t)bh * S * D;
    const uint16_t *Qh = a.Q + head_off, *Kh = a.K + head_off, *Vh = a.V + head_off;
    uint16_t *Oh = a.O + head_off;

    const int q0 = qblock * BR;
    const int qw = q0 + wave * 32;          // first query row of this wave
    const int my_q = qw + l32;              // query row on this lane
    const bool wave_live = qw < S;

    // Q^T fragments: B operand, lane = (query l32, head-dim slice 8*half..+7 of each 16)
    u32x4 qf[KS];
    if (wave_live) {
#pragma unroll
        for (int s = 0; s < KS; ++s)
            qf[s] = *reinterpret_cast<const u32x4 *>(Qh + (size_t)my_q * D + 16 * s + 8 * half);
    } else {
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = u32x4{0, 0, 0, 0};
    }

    int rows_in_block = S - q0 < BR ? S - q0 : BR;
    int tile_lo, tile_hi;
    fa_tile_range(S, kBlockKeys, a.L, a.R, q0, rows_in_block, &tile_lo, &tile_hi);

    // per-lane LDS read offsets (stage 0, key block 0 / slice 0)
    uint32_t koff[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s)
        koff[s] = (uint32_t)(l32 * ROWB + (((2 * s + half) ^ k_swz<CPR>(l32)) << 4));
    uint32_t voff[DB];
    {
        const int row0 = 4 * half + (l16 >> 2);
        const int dq = (l32 >> 4), c4 = l16 & 3;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const int c = 4 * db + 2 * dq + (c4 >> 1);
            voff[db] = (uint32_t)(TILEB + row0 * ROWB + ((c ^ v_swz<CPR>(row0)) << 4) + ((c4 & 1) << 3));
        }
    }

    // global -> register staging of the next tile
    u32x4 kreg[LPT], vreg[LPT];
    auto load_tile = [&](int tile) {
        const int k0 = tile * kBlockKeys;
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            const int P = tid + i * NT, row = P / CPR, pos = P % CPR;
            kreg[i] = *reinterpret_cast<const u32x4 *>(Kh + (size_t)(k0 + row) * D + ((pos ^ k_swz<CPR>(row)) << 3));
            vreg[i] = *reinterpret_cast<const u32x4 *>(Vh + (size_t)(k0 + row) * D + ((pos ^ v_swz<CPR>(row)) << 3));
        }
    };
    auto store_tile = [&](int stage) {
        const uint32_t base = lds0 + stage * 2 * TILEB;
#pragma unroll
        for (int i = 0; i < LPT; ++i) {
            const int P = tid + i * NT;
            lds_write_b128(base + P * 16, kreg[i]);
            lds_write_b128(base + TILEB + P * 16, vreg[i]);
        }
    };

    f32x16 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] = 0.0f;
    float m_run = -INFINITY;     // reference point of the exponentials, raw (unscaled) score units
    float l_run = 0.0f;          // this lane's half of the row sum
    const float c = a.scale_log2e;
    const float thresh = kRescaleLog2 / c;

    load_tile(tile_lo);
    store_tile(0);

    for (int tile = tile_lo; tile <= tile_hi; ++tile) {
        const int stage = (tile - tile_lo) & 1;
        if (tile < tile_hi) load_tile(tile + 1);
        __syncthreads();     // tile `tile` is visible; everyone is done with the other stage

        int cls = 2;
        if (MASKED) cls = fa_tile_class(kBlockKeys, a.L, a.R, qw, 32, tile);
        if (wave_live && cls != 0) {
            const uint32_t sbase = lds0 + stage * 2 * TILEB;
            // ---- S^T = K Q^T : two 32-key blocks
            f32x16 s0, s1;
#pragma unroll
            for (int r = 0; r < 16; ++r) { s0[r] = 0.0f; s1[r] = 0.0f; }
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const u32x4 ka = lds_read_b128(sbase + koff[s]);
                const u32x4 kb = lds_read_b128(sbase + koff[s] + 32 * ROWB);
                s0 = N::mfma(ka, qf[s], s0);
                s1 = N::mfma(kb, qf[s], s1);
            }
            // ---- mask (only on tiles that straddle an edge)
            if (MASKED && cls == 1) {
                const int kbase = tile * kBlockKeys + 4 * half;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int j0 = kbase + 8 * (r >> 2) + (r & 3);
                    const int j1 = j0 + 32;
                    if (j0 > my_q + a.R || j0 < my_q - a.L) s0[r] = -INFINITY;
                    if (j1 > my_q + a.R || j1 < my_q - a.L) s1[r] = -INFINITY;
                }
            }
            // ---- online softmax, lane-local over its 32 keys + one half-wave swap
            float mx = fmaxf(s0[0], s1[0]);
#pragma unroll
            for (int r = 1; r < 16; ++r) mx = fmaxf(fmaxf(mx, s0[r]), s1[r]);
            mx = fmaxf(mx, swap_halves(mx));
            const bool grow = mx > m_run + thresh;      // -inf + thresh = -inf: first finite max always grows
            if (__builtin_amdgcn_ballot_w64(grow) != 0) {
                const float m_new = grow ? mx : m_run;
                const float alpha = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m_run - m_new) * c);
                l_run *= alpha;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
                m_run = m_new;
            }
            const float mc = (m_run == -INFINITY) ? 0.0f : m_run * c;
            uint32_t p0[8], p1[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                p0[i] = N::pack2(__builtin_amdgcn_exp2f(__builtin_fmaf(s0[2 * i], c, -mc)),
                                 __builtin_amdgcn_exp2f(__builtin_fmaf(s0[2 * i + 1], c, -mc)));
                p1[i] = N::pack2(__builtin_amdgcn_exp2f(__builtin_fmaf(s1[2 * i], c, -mc)),
                                 __builtin_amdgcn_exp2f(__builtin_fmaf(s1[2 * i + 1], c, -mc)));
            }
#pragma unroll
            for (int i = 0; i < 8; ++i) { l_run = N::add_pair(p0[i], l_run); l_run = N::add_pair(p1[i], l_run); }
            // ---- O^T += V^T P^T : four 16-key slices x DB head-dim blocks
#pragma unroll
            for (int t2 = 0; t2 < 4; ++t2) {
                const uint32_t *pp = (t2 < 2) ? p0 : p1;
                const int tt = t2 & 1;
                const u32x4 pb = {pp[4 * tt], pp[4 * tt + 1], pp[4 * tt + 2], pp[4 * tt + 3]};
#pragma unroll
                for (int db = 0; db < DB; ++db) {
                    const u32x2 lo = lds_read_tr(sbase + voff[db] + (16 * t2) * ROWB);
                    const u32x2 hi = lds_read_tr(sbase + voff[db] + (16 * t2 + 8) * ROWB);
                    const u32x4 va = {lo[0], lo[1], hi[0], hi[1]};
                    o[db] = N::mfma(va, pb, o[db]);
                }
            }
        }
        if (tile < tile_hi) store_tile(stage ^ 1);
    }

    if (!wave_live) return;
    // ---- epilogue: O / l, logsumexp (the reference has none; flash_forward.h:318-327 only divides)
    const float l_tot = l_run + swap_halves(l_run);
    const float inv = 1.0f / l_tot;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 w;
            w[0] = N::pack2(o[db][4 * g] * inv, o[db][4 * g + 1] * inv);
            w[1] = N::pack2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
            *reinterpret_cast<u32x2 *>(Oh + (size_t)my_q * D + 32 * db + 8 * g + 4 * half) = w;
        }
    if (a.lse != nullptr && half == 0)
        a.lse[(size_t)bh * S + my_q] = m_run * a.scale + __builtin_logf(l_tot);
}


// ---------------------------------------------------------------------------
// Ping-pong variant: 8 waves, two per SIMD.  Waves 0-3 (group A) and 4-7
// (group B) run the same per-tile sequence  [MFMA phase: PV(t-1), QK(t)]
// [VALU phase: softmax(t)]  but B is one phase behind A, so on every SIMD one
// wave feeds the matrix core while the other does exp/max/convert.  The
// offset is made by one extra s_barrier in B's prologue; after that every
// wave executes one barrier per phase.  K/V tiles go global -> LDS directly
// (no VGPR staging), two stages each, issued two phases ahead of their use.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void wait_vm0() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// One wave-wide direct global->LDS load: lane l copies 16 bytes from base + voff (its own address) to
// LDS byte lds + 16*l.  Written as inline assembly so that the compiler does not order every later LDS
// read behind it with a vmcnt(0) wait; completion is waited for explicitly with wait_vm0() + barrier.
__device__ __forceinline__ void dma_16(const char *base, uint32_t voff, uint32_t lds)
{
    const uint64_t b = (uint64_t)base;     // wave-uniform by construction; say so, so that it lives in SGPRs
    // (readfirstlane returns a signed int: go through uint32_t, or the low half would sign-extend)
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint64_t ub = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds)), "v"(voff), "s"(ub) : "memory");
}
__device__ __forceinline__ void phase_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

#ifdef FA_PHASE_TIMING
// Development aid: per-wave cycle counts of the two phases and of the barrier waits.
#define FA_T(var) const long long var = (long long)__builtin_readcyclecounter()
#define FA_TACC(acc, t1, t0) acc += (t1) - (t0)
#else
#define FA_T(var)
#define FA_TACC(acc, t1, t0)
#endif

template <int V> struct IntC { static constexpr int value = V; };

template <bool BF16, int D, bool MASKED>
__global__ void __launch_bounds__(512) fa_fwd_pingpong(const FaKernelArgs a)
{
#ifdef FA_PHASE_TIMING
    long long tm_m = 0, tm_mw = 0, tm_x = 0, tm_xw = 0;
    const long long tm_begin = (long long)__builtin_readcyclecounter();
#endif
    constexpr int NW = 8;
    constexpr int BR = 32 * NW;
    constexpr int CPR = D / 8;
    constexpr int ROWB = D * 2;
    constexpr int TILEB = kBlockKeys * ROWB;
    constexpr int INSTR = TILEB / 1024;           // 1 KiB wave-wide direct-to-LDS loads per tile
    constexpr int IPW = INSTR / NW;               // ... per wave
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int NPV = 4 * DB;                   // PV matrix instructions per tile: (16-key slice, head-dim block)
    constexpr int NQK = 2 * KS;                   // QK matrix instructions per tile: (head-dim slice, 32-key block)
    constexpr int PD = 6;                         // LDS reads run this many matrix instructions ahead of their use
    constexpr uint32_t LDS_K = 0, LDS_V = 2 * TILEB;   // K stages at 0, TILEB; V stages at 2*TILEB, 3*TILEB
    static_assert(INSTR % NW == 0, "tile must divide over the waves");
    static_assert(4 * TILEB <= 65536, "stage offsets must fit the 16-bit LDS immediate");
    typedef Num<BF16> N;

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2;
    const int half = lane >> 5, l32 = lane & 31, l16 = lane & 15;

    int bh, qblock;
    fa_item_decode((long long)blockIdx.x, a.BH, a.n_qblocks, a.descending, &bh, &qblock);
    const int S = a.S;
    const size_t head_off = (size_t)bh * S * D;
    const uint16_t *Qh = a.Q + head_off, *Kh = a.K + head_off, *Vh = a.V + head_off;
    uint16_t *Oh = a.O + head_off;

    const int q0 = qblock * BR;
    const int qw = q0 + wave * 32;
    const int my_q = qw + l32;
    const bool wave_live = qw < S;

    u32x4 qf[KS];
    if (wave_live) {
#pragma unroll
        for (int s = 0; s < KS; ++s)
            qf[s] = *reinterpret_cast<const u32x4 *>(Qh + (size_t)my_q * D + 16 * s + 8 * half);
    } else {
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = u32x4{0, 0, 0, 0};
    }

    const int rows_in_block = S - q0 < BR ? S - q0 : BR;
    int tile_lo, tile_hi;
    fa_tile_range(S, kBlockKeys, a.L, a.R, q0, rows_in_block, &tile_lo, &tile_hi);

    // per-lane LDS read addresses for stage 0; stage, key block and key slice are immediates
    uint32_t koff[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s)
        koff[s] = lds0 + LDS_K + (uint32_t)(l32 * ROWB + (((2 * s + half) ^ k_swz<CPR>(l32)) << 4));
    uint32_t voff[DB];
    {
        const int row0 = 4 * half + (l16 >> 2);
        const int dq = (l32 >> 4), c4 = l16 & 3;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const int c = 4 * db + 2 * dq + (c4 >> 1);
            voff[db] = lds0 + LDS_V + (uint32_t)(row0 * ROWB + ((c ^ v_swz<CPR>(row0)) << 4) + ((c4 & 1) << 3));
        }
    }

    // direct global -> LDS tile loads: wave w issues instructions w, w+8, ... of the tile; instruction n
    // fills LDS bytes [n*1024, n*1024+1024) linearly, lane l supplying the swizzled source chunk.
    uint32_t gk[IPW], gv[IPW];
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
        const int P = (i * NW + wave) * 64 + lane, row = P / CPR, pos = P % CPR;
        gk[i] = (uint32_t)(row * ROWB + ((pos ^ k_swz<CPR>(row)) << 4));
        gv[i] = (uint32_t)(row * ROWB + ((pos ^ v_swz<CPR>(row)) << 4));
    }
    auto issue_k = [&](int tile, int stage) __attribute__((always_inline)) {
        const char *src = reinterpret_cast<const char *>(Kh) + (size_t)tile * TILEB;
#pragma unroll
        for (int i = 0; i < IPW; ++i) dma_16(src, gk[i], lds0 + LDS_K + stage * TILEB + (i * NW + wave) * 1024);
    };
    auto issue_v = [&](int tile, int stage) __attribute__((always_inline)) {
        const char *src = reinterpret_cast<const char *>(Vh) + (size_t)tile * TILEB;
#pragma unroll
        for (int i = 0; i < IPW; ++i) dma_16(src, gv[i], lds0 + LDS_V + stage * TILEB + (i * NW + wave) * 1024);
    };

    f32x16 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;
    const float c = a.scale_log2e;
    const float thresh = kRescaleLog2 / c;
    uint32_t p0[8], p1[8];
    f32x16 s0, s1;
    bool have_p = false;

    // O^T += V^T P^T from V stage VS, software-pipelined: each transposed LDS read is issued PD matrix
    // instructions before its use; scheduling barriers keep the compiler from folding them back together.
    auto pv = [&](auto VS) __attribute__((always_inline)) {
        constexpr uint32_t vs = decltype(VS)::value * TILEB;
        u32x4 vfr[NPV];
        auto read_v = [&](int n) __attribute__((always_inline)) {
            const int t2 = n / DB, db = n % DB;
            const u32x2 lo = lds_read_tr(voff[db] + vs + (16 * t2) * ROWB);
            const u32x2 hi = lds_read_tr(voff[db] + vs + (16 * t2 + 8) * ROWB);
            return u32x4{lo[0], lo[1], hi[0], hi[1]};
        };
#pragma unroll
        for (int n = 0; n < PD; ++n) vfr[n] = read_v(n);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = 0; n < NPV; ++n) {
            if (n + PD < NPV) vfr[n + PD] = read_v(n + PD);
            const int t2 = n / DB, db = n % DB;
            const uint32_t *pp = (t2 < 2) ? p0 : p1;
            const int tt = t2 & 1;
            const u32x4 pb = {pp[4 * tt], pp[4 * tt + 1], pp[4 * tt + 2], pp[4 * tt + 3]};
            o[db] = N::mfma(vfr[n], pb, o[db]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // S^T = K Q^T from K stage KSTG, pipelined the same way
    auto qk = [&](auto KSTG) __attribute__((always_inline)) {
        constexpr uint32_t ks = decltype(KSTG)::value * TILEB;
        u32x4 kfr[NQK];
        auto read_k = [&](int n) __attribute__((always_inline)) { return lds_read_b128(koff[n >> 1] + ks + (n & 1) * 32 * ROWB); };
#pragma unroll
        for (int n = 0; n < PD; ++n) kfr[n] = read_k(n);
#pragma unroll
        for (int r = 0; r < 16; ++r) { s0[r] = 0.0f; s1[r] = 0.0f; }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = 0; n < NQK; ++n) {
            if (n + PD < NQK) kfr[n + PD] = read_k(n + PD);
            if (n & 1) s1 = N::mfma(kfr[n], qf[n >> 1], s1);
            else s0 = N::mfma(kfr[n], qf[n >> 1], s0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    auto softmax = [&](int tile, int cls) __attribute__((always_inline)) {
        if (MASKED && cls == 1) {
            const int kb0 = tile * kBlockKeys + 4 * half;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int j0 = kb0 + 8 * (r >> 2) + (r & 3);
                const int j1 = j0 + 32;
                if (j0 > my_q + a.R || j0 < my_q - a.L) s0[r] = -INFINITY;
                if (j1 > my_q + a.R || j1 < my_q - a.L) s1[r] = -INFINITY;
            }
        }
        float mx = fmaxf(s0[0], s1[0]);
#pragma unroll
        for (int r = 1; r < 16; ++r) mx = fmaxf(fmaxf(mx, s0[r]), s1[r]);
        mx = fmaxf(mx, swap_halves(mx));
        const bool grow = mx > m_run + thresh;      // -inf + thresh = -inf: a first finite max always grows
        if (__builtin_amdgcn_ballot_w64(grow) != 0) {
            const float m_new = grow ? mx : m_run;
            const float alpha = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m_run - m_new) * c);
            l_run *= alpha;
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
            m_run = m_new;
        }
        const float mc = (m_run == -INFINITY) ? 0.0f : m_run * c;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            p0[i] = N::pack2(__builtin_amdgcn_exp2f(__builtin_fmaf(s0[2 * i], c, -mc)),
                             __builtin_amdgcn_exp2f(__builtin_fmaf(s0[2 * i + 1], c, -mc)));
            p1[i] = N::pack2(__builtin_amdgcn_exp2f(__builtin_fmaf(s1[2 * i], c, -mc)),
                             __builtin_amdgcn_exp2f(__builtin_fmaf(s1[2 * i + 1], c, -mc)));
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) { l_run = N::add_pair(p0[i], l_run); l_run = N::add_pair(p1[i], l_run); }
    };

    // One tile: [MFMA phase: PV(tile-1) from V stage BUF^1, QK(tile) from K stage BUF] barrier
    //           [VALU phase: softmax(tile)] barrier.  BUF is a compile-time constant so that every LDS
    // address is a register plus an immediate.
    auto step = [&](auto BUF, int tile) __attribute__((always_inline)) {
        constexpr int buf = decltype(BUF)::value;
        int cls = 2;
        if (MASKED) cls = fa_tile_class(kBlockKeys, a.L, a.R, qw, 32, tile);
        const bool active = wave_live && cls != 0;
        FA_T(t_a);
        if (grp == 0) {                       // A issues its share of the loads for two phases from now
            if (tile < tile_hi) issue_k(tile + 1, buf ^ 1);
            issue_v(tile, buf);
        }
        if (have_p) pv(IntC<buf ^ 1>{});
        if (active) qk(IntC<buf>{});
        FA_T(t_b);
        if (grp == 1) wait_vm0();
        phase_barrier();
        FA_T(t_c);
        if (grp == 1) {                       // B does the same one phase later
            if (tile + 2 <= tile_hi) issue_k(tile + 2, buf);
            if (tile + 1 <= tile_hi) issue_v(tile + 1, buf ^ 1);
        }
        have_p = active;
        if (active) softmax(tile, cls);
        FA_T(t_d);
        if (grp == 0) wait_vm0();
        phase_barrier();
        FA_T(t_e);
        FA_TACC(tm_m, t_b, t_a); FA_TACC(tm_mw, t_c, t_b); FA_TACC(tm_x, t_d, t_c); FA_TACC(tm_xw, t_e, t_d);
    };

    // ---- prologue
    issue_k(tile_lo, 0);
    wait_vm0();
    // the Q fragments have landed (vmcnt is 0); touching them here lets the compiler see that as well, so it
    // places no vmcnt wait inside the loop, where it would also wait for the asynchronous tile loads
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]));
    phase_barrier();
    if (grp == 1) {           // B idles through A's first MFMA phase, but issues its share of the loads
        if (tile_lo < tile_hi) issue_k(tile_lo + 1, 1);
        issue_v(tile_lo, 0);
        phase_barrier();
    }

    for (int tile = tile_lo; tile <= tile_hi; tile += 2) {
        step(IntC<0>{}, tile);
        if (tile + 1 <= tile_hi) step(IntC<1>{}, tile + 1);
    }
    // ---- drain: PV of the last tile; A executes the barrier B spent in its prologue
    if (have_p) {
        if ((tile_hi - tile_lo) & 1) pv(IntC<1>{});
        else pv(IntC<0>{});
    }
    if (grp == 0) phase_barrier();

    if (!wave_live) return;
    const float l_tot = l_run + swap_halves(l_run);
    const float inv = 1.0f / l_tot;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 w;
            w[0] = N::pack2(o[db][4 * g] * inv, o[db][4 * g + 1] * inv);
            w[1] = N::pack2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
            *reinterpret_cast<u32x2 *>(Oh + (size_t)my_q * D + 32 * db + 8 * g + 4 * half) = w;
        }
    if (a.lse != nullptr && half == 0)
        a.lse[(size_t)bh * S + my_q] = m_run * a.scale + __builtin_logf(l_tot);
#ifdef FA_PHASE_TIMING
    if (a.dbg != nullptr && lane == 0) {
        long long *d = a.dbg + ((size_t)blockIdx.x * NW + wave) * 8;
        d[0] = tm_m; d[1] = tm_mw; d[2] = tm_x; d[3] = tm_xw;
        d[4] = (long long)__builtin_readcyclecounter() - tm_begin; d[5] = tile_hi - tile_lo + 1;
        d[6] = (long long)wall_clock64();
    }
#endif
}



// ---------------------------------------------------------------------------
// Software-pipelined variant.  Every wave runs ONE instruction stream per key
// tile in which the matrix instructions of PV(tile-1) and QK(tile+1) are
// interleaved, a few vector instructions at a time, with the softmax of
// `tile`: a single wave keeps the matrix core busy while its own exp/max/
// convert work issues in the gaps, and the second wave on the SIMD fills
// whatever is left.  K/V tiles stream global -> LDS directly through three
// stages each, issued two iterations before their first use; one workgroup
// barrier per tile.
// ---------------------------------------------------------------------------
template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }

template <bool BF16, int D, bool MASKED>
__global__ void __launch_bounds__(512) fa_fwd_pipelined(const FaKernelArgs a)
{
#ifdef FA_PHASE_TIMING
    long long tm_m = 0, tm_mw = 0, tm_x = 0, tm_xw = 0, tm_n = 0;
    const long long tm_begin = (long long)__builtin_readcyclecounter();
    const long long tw_begin = (long long)wall_clock64();
#endif
    constexpr int NW = 8;
    constexpr int BR = 32 * NW;
    constexpr int CPR = D / 8;
    constexpr int ROWB = D * 2;
    constexpr int TILEB = kBlockKeys * ROWB;
    constexpr int INSTR = TILEB / 1024;
    constexpr int IPW = INSTR / NW;               // direct-to-LDS instructions per wave per tile
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int NPV = 4 * DB;                   // PV matrix instructions per tile
    constexpr int NQK = 2 * KS;                   // QK matrix instructions per tile
    constexpr int NM = NPV + NQK;
    constexpr int PD = 6;                         // LDS reads run this many matrix instructions ahead
    constexpr int NST = 3;                        // LDS stages per tensor
    constexpr uint32_t LDS_V = NST * TILEB;       // K stages first, then V stages
    static_assert(INSTR % NW == 0, "tile must divide over the waves");
    static_assert(NST * TILEB <= 65536, "stage offsets must fit the 16-bit LDS immediate");
    typedef Num<BF16> N;

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, l32 = lane & 31, l16 = lane & 15;

    int bh, qblock;
    fa_item_decode((long long)blockIdx.x, a.BH, a.n_qblocks, a.descending, &bh, &qblock);
    const int S = a.S;
    const size_t head_off = (size_t)bh * S * D;
    const uint16_t *Qh = a.Q + head_off, *Kh = a.K + head_off, *Vh = a.V + head_off;
    uint16_t *Oh = a.O + head_off;

    const int q0 = qblock * BR;
    const int qw = q0 + wave * 32;
    const int my_q = qw + l32;
    const bool wave_live = qw < S;

    u32x4 qf[KS];
    if (wave_live) {
#pragma unroll
        for (int s = 0; s < KS; ++s)
            qf[s] = *reinterpret_cast<const u32x4 *>(Qh + (size_t)my_q * D + 16 * s + 8 * half);
    } else {
#pragma unroll
        for (int s = 0; s < KS; ++s) qf[s] = u32x4{0, 0, 0, 0};
    }

    const int rows_in_block = S - q0 < BR ? S - q0 : BR;
    int t0, t1;                 // key tiles visited by the workgroup
    fa_tile_range(S, kBlockKeys, a.L, a.R, q0, rows_in_block, &t0, &t1);
    int my_lo = 1, my_hi = 0;   // key tiles with at least one visible pair for this wave (contiguous)
    if (wave_live) fa_tile_range(S, kBlockKeys, a.L, a.R, qw, 32, &my_lo, &my_hi);

    uint32_t koff[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s)
        koff[s] = lds0 + (uint32_t)(l32 * ROWB + (((2 * s + half) ^ k_swz<CPR>(l32)) << 4));
    uint32_t voff[DB];
    {
        const int row0 = 4 * half + (l16 >> 2);
        const int dq = (l32 >> 4), c4 = l16 & 3;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const int c = 4 * db + 2 * dq + (c4 >> 1);
            voff[db] = lds0 + LDS_V + (uint32_t)(row0 * ROWB + ((c ^ v_swz<CPR>(row0)) << 4) + ((c4 & 1) << 3));
        }
    }
    uint32_t gk[IPW], gv[IPW];
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
        const int P = (i * NW + wave) * 64 + lane, row = P / CPR, pos = P % CPR;
        gk[i] = (uint32_t)(row * ROWB + ((pos ^ k_swz<CPR>(row)) << 4));
        gv[i] = (uint32_t)(row * ROWB + ((pos ^ v_swz<CPR>(row)) << 4));
    }
    auto issue_k = [&](int tile, int stage) __attribute__((always_inline)) {
        const char *src = reinterpret_cast<const char *>(Kh) + (size_t)tile * TILEB;
#pragma unroll
        for (int i = 0; i < IPW; ++i) dma_16(src, gk[i], lds0 + stage * TILEB + (i * NW + wave) * 1024);
    };
    auto issue_v = [&](int tile, int stage) __attribute__((always_inline)) {
        const char *src = reinterpret_cast<const char *>(Vh) + (size_t)tile * TILEB;
#pragma unroll
        for (int i = 0; i < IPW; ++i) dma_16(src, gv[i], lds0 + LDS_V + stage * TILEB + (i * NW + wave) * 1024);
    };

    f32x16 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] = 0.0f;
    float m_run = -INFINITY, l_a = 0.0f, l_b = 0.0f;
    const float c = a.scale_log2e;
    const float thresh = kRescaleLog2 / c;
    uint32_t pk[16];            // P of the tile whose PV comes next: [0..7] keys 0..31, [8..15] keys 32..63
    f32x16 s0, s1;              // S^T of the tile whose softmax comes next

    auto read_v = [&](uint32_t vs, int n) __attribute__((always_inline)) {
        const int t2 = n / DB, db = n % DB;
        const u32x2 lo = lds_read_tr(voff[db] + vs + (16 * t2) * ROWB);
        const u32x2 hi = lds_read_tr(voff[db] + vs + (16 * t2 + 8) * ROWB);
        return u32x4{lo[0], lo[1], hi[0], hi[1]};
    };
    auto read_k = [&](uint32_t ks, int n) __attribute__((always_inline)) {
        return lds_read_b128(koff[n >> 1] + ks + (n & 1) * 32 * ROWB);
    };
    auto apply_mask = [&](int tile) __attribute__((always_inline)) {
        const int kb0 = tile * kBlockKeys + 4 * half;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int j0 = kb0 + 8 * (r >> 2) + (r & 3);
            const int j1 = j0 + 32;
            if (j0 > my_q + a.R || j0 < my_q - a.L) s0[r] = -INFINITY;
            if (j1 > my_q + a.R || j1 < my_q - a.L) s1[r] = -INFINITY;
        }
    };
    // row maximum of S(tile) and the decision to move the reference point; returns the factor by which
    // everything accumulated so far has to be multiplied (1 when the reference point stays)
    auto new_reference = [&](float mx, bool &moved) __attribute__((always_inline)) {
        float alpha = 1.0f;
        const bool grow = mx > m_run + thresh;      // -inf + thresh = -inf: a first finite max always grows
        moved = __builtin_amdgcn_ballot_w64(grow) != 0;
        if (moved) {
            const float m_new = grow ? mx : m_run;
            alpha = (m_run == -INFINITY) ? 0.0f : __builtin_amdgcn_exp2f((m_run - m_new) * c);
            l_a *= alpha;
            l_b *= alpha;
            m_run = m_new;
        }
        return alpha;
    };
    auto scale_o = [&](float alpha) __attribute__((always_inline)) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
    };

    // ---- plain (not interleaved) pieces, used while the pipeline fills and drains
    // (the scheduling barriers keep register pressure low here: without them the compiler hoists every
    // LDS read of the unrolled loop to the top and spills)
    auto pv_plain = [&](int vstage) __attribute__((always_inline)) {
        const uint32_t vs = vstage * TILEB;
        u32x4 fr[NPV];
        fr[0] = read_v(vs, 0);
        fr[1] = read_v(vs, 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = 0; n < NPV; ++n) {
            if (n + 2 < NPV) fr[n + 2] = read_v(vs, n + 2);
            const int t2 = n / DB, db = n % DB;
            const u32x4 pb = {pk[4 * t2], pk[4 * t2 + 1], pk[4 * t2 + 2], pk[4 * t2 + 3]};
            o[db] = N::mfma(fr[n], pb, o[db]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto qk_plain = [&](int kstage) __attribute__((always_inline)) {
        const uint32_t ks = kstage * TILEB;
        u32x4 fr[NQK];
        fr[0] = read_k(ks, 0);
        fr[1] = read_k(ks, 1);
#pragma unroll
        for (int r = 0; r < 16; ++r) { s0[r] = 0.0f; s1[r] = 0.0f; }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = 0; n < NQK; ++n) {
            if (n + 2 < NQK) fr[n + 2] = read_k(ks, n + 2);
            if (n & 1) s1 = N::mfma(fr[n], qf[n >> 1], s1);
            else s0 = N::mfma(fr[n], qf[n >> 1], s0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto softmax_plain = [&](int tile) __attribute__((always_inline)) {
        if (MASKED && fa_tile_class(kBlockKeys, a.L, a.R, qw, 32, tile) == 1) apply_mask(tile);
        float mx = fmaxf(s0[0], s1[0]);
#pragma unroll
        for (int r = 1; r < 16; ++r) mx = fmaxf(fmaxf(mx, s0[r]), s1[r]);
        mx = fmaxf(mx, swap_halves(mx));
        bool moved;
        const float alpha = new_reference(mx, moved);
        if (moved) scale_o(alpha);
        const float mc = (m_run == -INFINITY) ? 0.0f : m_run * c;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s0[2 * i], c, -mc));
            const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s0[2 * i + 1], c, -mc));
            const float e2 = __builtin_amdgcn_exp2f(__builtin_fmaf(s1[2 * i], c, -mc));
            const float e3 = __builtin_amdgcn_exp2f(__builtin_fmaf(s1[2 * i + 1], c, -mc));
            l_a += e0; l_b += e1; l_a += e2; l_b += e3;
            pk[i] = N::pack2(e0, e1);
            pk[8 + i] = N::pack2(e2, e3);
        }
    };

    // ---- the steady-state iteration: PV(tile-1) from V stage VST, softmax(tile), QK(tile+1) from K stage KST
    auto steady = [&](auto KST, auto VST, int tile) __attribute__((always_inline)) {
        constexpr uint32_t ks = decltype(KST)::value * TILEB;
        constexpr uint32_t vs = decltype(VST)::value * TILEB;
        u32x4 fr[NM];                              // operand fragments, in matrix-instruction order
        auto fetch = [&](int n) __attribute__((always_inline)) {
#ifdef FA_EXP_NO_LDS
            fr[n] = qf[n % KS];
#else
            if (n < NPV) fr[n] = read_v(vs, n);
            else fr[n] = read_k(ks, n - NPV);
#endif
        };
#pragma unroll
        for (int n = 0; n < PD; ++n) fetch(n);
        // the fragments are in flight; the row maximum needs no matrix instruction and covers their latency
        if (MASKED && fa_tile_class(kBlockKeys, a.L, a.R, qw, 32, tile) == 1) apply_mask(tile);
        float mx = fmaxf(s0[0], s1[0]);
#pragma unroll
        for (int r = 1; r < 16; ++r) mx = fmaxf(fmaxf(mx, s0[r]), s1[r]);
        mx = fmaxf(mx, swap_halves(mx));
        bool moved;
        const float alpha = new_reference(mx, moved);
        const float mc = (m_run == -INFINITY) ? 0.0f : m_run * c;
        uint32_t pn[16];                           // P(tile), becomes pk at the end
        f32x16 n0, n1;                             // S^T(tile+1)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < NM; ++g) {
            if (g + PD < NM) fetch(g + PD);
            if (g < NPV) {
                const int t2 = g / DB, db = g % DB;
                const u32x4 pb = {pk[4 * t2], pk[4 * t2 + 1], pk[4 * t2 + 2], pk[4 * t2 + 3]};
                o[db] = N::mfma(fr[g], pb, o[db]);
            } else {
                const int n = g - NPV;
                const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                if (n & 1) n1 = N::mfma(fr[g], qf[n >> 1], n < 2 ? zero : n1);
                else n0 = N::mfma(fr[g], qf[n >> 1], n < 2 ? zero : n0);
            }
            // softmax work riding along: 16 element pairs spread over the NM matrix instructions
            constexpr int PAIRS = 16;
            const int e_begin = (g * PAIRS) / NM, e_end = ((g + 1) * PAIRS) / NM;
#ifdef FA_EXP_NO_VALU
            for (int e = e_begin; e < e_end; ++e) pn[e] = pk[e];
#else
#pragma unroll
            for (int e = e_begin; e < e_end; ++e) {
                // pair e: elements (2e, 2e+1) of s0 for e < 8, of s1 for e >= 8.  The two empty asm
                // statements pin the arithmetic between the surrounding matrix instructions: without them
                // the compiler sinks all of it to the end of the iteration.
                float x0 = e < 8 ? s0[2 * e] : s1[2 * (e - 8)];
                float x1 = e < 8 ? s0[2 * e + 1] : s1[2 * (e - 8) + 1];
                asm volatile("" : "+v"(x0), "+v"(x1));
                const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(x0, c, -mc));
                const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(x1, c, -mc));
                l_a += e0;
                l_b += e1;
                uint32_t packed = N::pack2(e0, e1);
                asm volatile("" : "+v"(packed), "+v"(l_a), "+v"(l_b));
                pn[e] = packed;
            }
#endif
            __builtin_amdgcn_sched_barrier(0);
        }
        if (moved) scale_o(alpha);                 // rare; PV(tile-1) has been issued in full by now
#pragma unroll
        for (int i = 0; i < 16; ++i) pk[i] = pn[i];
        s0 = n0;
        s1 = n1;
    };

    // ---- prologue: K(t0) and K(t0+1) resident before the first iteration
    issue_k(t0, 0);
    if (t0 + 1 <= t1) issue_k(t0 + 1, 1);
    wait_vm<0>();
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]));   // Q has landed; see the note in the ping-pong kernel
    phase_barrier();

    // Iteration j (tile i = t0 - 1 + j) does PV(i-1), softmax(i), QK(i+1); it reads K stage j % 3 and V stage
    // (j + 1) % 3, and issues the loads of K(i+3) into K stage (j + 2) % 3 and of V(i+1) into V stage j % 3.
    // Every wave executes every iteration (one barrier each); a wave whose own tile range does not cover all
    // three pieces runs the plain pieces it has, the others run the interleaved body.  The two kinds live in
    // separate loops: merging them under one branch makes the register allocator spill.
    auto finish_iteration = [&](bool more_k, bool more_v) __attribute__((always_inline)) {
        // loads issued one iteration ago must have landed; those issued just now may stay in flight
        if (more_k && more_v) wait_vm<2 * IPW>();
        else wait_vm<0>();
        phase_barrier();
    };
    auto generic_iteration = [&](int i, int j3) __attribute__((always_inline)) {
        const bool more_k = i + 3 <= t1, more_v = i + 1 <= t1;
        const int j3p1 = j3 == NST - 1 ? 0 : j3 + 1, j3p2 = j3p1 == NST - 1 ? 0 : j3p1 + 1;
        FA_T(t_a);
        if (more_k) issue_k(i + 3, j3p2);
        if (more_v) issue_v(i + 1, j3);
        if (my_lo <= i - 1 && i - 1 <= my_hi) pv_plain(j3p1);
        if (my_lo <= i && i <= my_hi) softmax_plain(i);
        if (my_lo <= i + 1 && i + 1 <= my_hi) qk_plain(j3);
        FA_T(t_b);
        finish_iteration(more_k, more_v);
        FA_T(t_c);
        FA_TACC(tm_x, t_b, t_a); FA_TACC(tm_xw, t_c, t_b);
    };
    auto steady_iteration = [&](auto J3, int i) __attribute__((always_inline)) {
        constexpr int j3 = decltype(J3)::value;
        const bool more_k = i + 3 <= t1, more_v = i + 1 <= t1;
#ifndef FA_EXP_NO_DMA
        if (more_k) issue_k(i + 3, (j3 + 2) % NST);
        if (more_v) issue_v(i + 1, j3);
#endif
        FA_T(t_a);
        steady(IntC<j3>{}, IntC<(j3 + 1) % NST>{}, i);
        FA_T(t_b);
        finish_iteration(more_k, more_v);
        FA_T(t_c);
        FA_TACC(tm_m, t_b, t_a); FA_TACC(tm_mw, t_c, t_b);
#ifdef FA_PHASE_TIMING
        tm_n += 1;
#endif
    };
#ifdef FA_PHASE_TIMING
    const long long tm_loop0 = (long long)__builtin_readcyclecounter();
#endif
    int i = t0 - 1, j3 = 0;
    for (; i <= t1 + 1; ++i) {            // fill: until three consecutive iterations are steady and the stage is 0
        if (j3 == 0 && i >= my_lo + 1 && i + 2 <= my_hi - 1) break;
        generic_iteration(i, j3);
        j3 = j3 == NST - 1 ? 0 : j3 + 1;
    }
    for (; i >= my_lo + 1 && i + 2 <= my_hi - 1 && i <= t1 + 1; i += 3) {
        steady_iteration(IntC<0>{}, i);
        steady_iteration(IntC<1>{}, i + 1);
        steady_iteration(IntC<2>{}, i + 2);
    }
    for (j3 = 0; i <= t1 + 1; ++i) {      // drain
        generic_iteration(i, j3);
        j3 = j3 == NST - 1 ? 0 : j3 + 1;
    }

#ifdef FA_PHASE_TIMING
    const long long tm_loop1 = (long long)__builtin_readcyclecounter();
#endif
    if (!wave_live) return;
    const float l_half = l_a + l_b;
    const float l_tot = l_half + swap_halves(l_half);
    const float inv = 1.0f / l_tot;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 w;
            w[0] = N::pack2(o[db][4 * g] * inv, o[db][4 * g + 1] * inv);
            w[1] = N::pack2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
            *reinterpret_cast<u32x2 *>(Oh + (size_t)my_q * D + 32 * db + 8 * g + 4 * half) = w;
        }
    if (a.lse != nullptr && half == 0)
        a.lse[(size_t)bh * S + my_q] = m_run * a.scale + __builtin_logf(l_tot);
#ifdef FA_PHASE_TIMING
    if (a.dbg != nullptr && lane == 0) {
        long long *d = a.dbg + ((size_t)blockIdx.x * NW + wave) * 8;
        d[0] = tm_m; d[1] = tm_mw; d[2] = tm_x; d[3] = tm_xw;
        d[4] = (long long)__builtin_readcyclecounter() - tm_begin; d[5] = (t1 - t0 + 1) | (((long long)wall_clock64() - tw_begin) << 32);
        d[6] = ((tm_loop0 - tm_begin) << 32) | (((long long)__builtin_readcyclecounter() - tm_loop1) & 0xffffffffLL); d[7] = tm_n;
    }
#endif
}

}  // namespace

template <bool BF16, int D, int NW, bool MASKED>
static hipError_t launch_one(const FaKernelArgs &a, long long n_items, hipStream_t stream)
{
    constexpr int TILEB = kBlockKeys * D * 2;
    const size_t smem = 2 * 2 * TILEB;
    auto kern = fa_fwd_kernel<BF16, D, NW, MASKED>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)n_items), dim3(NW * 64), smem, stream, a);
    return hipGetLastError();
}

template <bool BF16, int D, bool MASKED>
static hipError_t launch_pingpong(const FaKernelArgs &a, long long n_items, hipStream_t stream)
{
    constexpr int TILEB = kBlockKeys * D * 2;
    const size_t smem = 4 * TILEB;
    auto kern = fa_fwd_pingpong<BF16, D, MASKED>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)n_items), dim3(512), smem, stream, a);
    return hipGetLastError();
}

template <bool BF16, int D, bool MASKED>
static hipError_t launch_pipelined(const FaKernelArgs &a, long long n_items, hipStream_t stream)
{
    constexpr int TILEB = kBlockKeys * D * 2;
    const size_t smem = 6 * TILEB;
    auto kern = fa_fwd_pipelined<BF16, D, MASKED>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kern, dim3((unsigned)n_items), dim3(512), smem, stream, a);
    return hipGetLastError();
}

hipError_t fa_launch_forward(const FaKernelArgs &a, int bf16, int D, int masked, long long n_items, hipStream_t stream)
{
    static const int variant = getenv("FA_FWD_VARIANT") ? atoi(getenv("FA_FWD_VARIANT")) : 3;
    if (variant == 3) {
#define FA_PL(BF, DD, MK) \
    if (bf16 == BF && D == DD && masked == MK) return launch_pipelined<BF != 0, DD, MK != 0>(a, n_items, stream);
        FA_PL(0, 64, 0) FA_PL(0, 64, 1) FA_PL(0, 128, 0) FA_PL(0, 128, 1)
        FA_PL(1, 64, 0) FA_PL(1, 64, 1) FA_PL(1, 128, 0) FA_PL(1, 128, 1)
#undef FA_PL
    }
    if (variant == 2) {
#define FA_PP(BF, DD, MK) \
    if (bf16 == BF && D == DD && masked == MK) return launch_pingpong<BF != 0, DD, MK != 0>(a, n_items, stream);
        FA_PP(0, 64, 0) FA_PP(0, 64, 1) FA_PP(0, 128, 0) FA_PP(0, 128, 1)
        FA_PP(1, 64, 0) FA_PP(1, 64, 1) FA_PP(1, 128, 0) FA_PP(1, 128, 1)
#undef FA_PP
    }
#define FA_CASE(BF, DD, MK) \
    if (bf16 == BF && D == DD && masked == MK) return launch_one<BF != 0, DD, 8, MK != 0>(a, n_items, stream);
    FA_CASE(0, 64, 0) FA_CASE(0, 64, 1) FA_CASE(0, 128, 0) FA_CASE(0, 128, 1)
    FA_CASE(1, 64, 0) FA_CASE(1, 64, 1) FA_CASE(1, 128, 0) FA_CASE(1, 128, 1)
#undef FA_CASE
    return hipErrorInvalidValue;
}
