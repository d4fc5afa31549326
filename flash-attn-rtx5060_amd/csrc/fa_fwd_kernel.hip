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

hipError_t fa_launch_forward(const FaKernelArgs &a, int bf16, int D, int masked, long long n_items, hipStream_t stream)
{
#define FA_CASE(BF, DD, MK) \
    if (bf16 == BF && D == DD && masked == MK) return launch_one<BF != 0, DD, 8, MK != 0>(a, n_items, stream);
    FA_CASE(0, 64, 0) FA_CASE(0, 64, 1) FA_CASE(0, 128, 0) FA_CASE(0, 128, 1)
    FA_CASE(1, 64, 0) FA_CASE(1, 64, 1) FA_CASE(1, 128, 0) FA_CASE(1, 128, 1)
#undef FA_CASE
    return hipErrorInvalidValue;
}
