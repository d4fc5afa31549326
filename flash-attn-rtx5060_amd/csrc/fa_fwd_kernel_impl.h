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
//  * K/V tiles go global -> LDS directly (global_load_lds_dwordx4, the role of
//    the TMA loads at include/utils.h:86-99), XOR-swizzled at 16-byte
//    granularity on the global-address side so that both the ds_read_b128
//    K-operand pattern and the transposed V pattern are free of bank conflicts
//    without padding (the reference tiles are unswizzled, utils.h:168).  Two or
//    three LDS stages per tensor replace the mbarrier ring (flash_forward.h:95-111).
//  * Software pipelining inside every wave: the matrix instructions of
//    PV(tile-1) and QK(tile+1) are interleaved, a few vector instructions at a
//    time, with the softmax of `tile`, so the matrix core stays busy while the
//    wave's own exp/max/convert work issues in the gaps (the reference runs
//    QK, softmax and PV back to back, flash_forward.h:193-315).
//  * exp2 with scale*log2(e) folded into one FMA, the rescale of O done only
//    when a row maximum has grown by more than 2^8 (the reference recomputes
//    the factor 4*d/8 times per tile, flash_forward.h:296-299), the -inf
//    guard the reference lacks (softmax.h:55,83).
//  * Masks are evaluated per element only on tiles that straddle a mask edge,
//    and tiles that are fully masked for a wave are skipped by that wave (the
//    reference masks every tile, mask.h:10-84).
//  * Work items (batch*head, query block) are either dispatched one per
//    workgroup in longest-first order, or walked by a persistent grid of one
//    workgroup per CU in a snake over the same list (Schedule<0,...>,
//    flash_forward.h:22-65, walks it round-robin in natural order).
#ifndef FA_FWD_KERNEL_IMPL_H
#define FA_FWD_KERNEL_IMPL_H
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "fa_device_state.h"
#include "fa_kernel_args.h"
#include "fa_sched.h"

// The row maximum of a tile's scores is taken next to this many of the iteration's first matrix instructions
// (0: in front of them).
#ifndef FA_S1K
#define FA_S1K 3
#define FA_S1V 2
#endif
#ifndef FA_ROW_MAX_SLOTS
#define FA_ROW_MAX_SLOTS 4
#endif

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kBlockKeys = 64;          // keys per K/V tile
constexpr float kNoReference = -1.0e30f; // reference point of a row before its first visible score
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
};

// 16-byte-chunk swizzles.  A tile row holds CPR = D/8 chunks.
// K is read with ds_read_b128 by 16 lanes holding 16 consecutive rows and one
// logical chunk: those must land on 16 different 16-byte bank groups.
template <int CPR> __device__ __forceinline__ int k_swz(int row) { return CPR == 16 ? (row & 15) : ((row >> 1) & 7); }
// V is read with ds_read_b64_tr_b16: 32 lanes cover 4 consecutive rows x 4
// consecutive chunks; the 4 rows must land on 4 different 64-byte bank groups.
template <int CPR> __device__ __forceinline__ int v_swz(int row) { return CPR == 16 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2); }

// max(x of lane l, x of lane l^32), in both lanes: after v_permlane32_swap of two copies one register holds the
// lower half's values in both halves and the other the upper half's.  (The maximum as an instruction of its own:
// written as fmaxf the compiler first quiets possible signalling NaNs in both operands, an instruction each.)
__device__ __forceinline__ float max_plain(float a, float b)
{
    float m;
    asm("v_max_f32 %0, %1, %2" : "=v"(m) : "v"(a), "v"(b));
    return m;
}
// (One assembly statement: handed the two results of __builtin_amdgcn_permlane32_swap, an inline-assembly
// v_max_f32 received the first of them twice (hipcc 7.2).  The s_nop covers the wait states the swap needs
// behind the vector instructions that wrote its operands.)
__device__ __forceinline__ float max_of_halves(float x)
{
    float a = x, b = x, m;
    asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\tv_max_f32 %2, %0, %1" : "+v"(a), "+v"(b), "=v"(m));
    return m;
}
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

// One wave-wide direct global->LDS load: lane l copies 16 bytes from base + voff (its own address) to
// LDS byte lds + 16*l.  Written as inline assembly so that the compiler does not order every later LDS
// read behind it with a vmcnt(0) wait; completion is waited for explicitly with s_waitcnt vmcnt + barrier.
__device__ __forceinline__ void dma_16(const char *base, uint32_t voff, uint32_t lds)
{
    const uint64_t b = (uint64_t)base;     // wave-uniform by construction; say so, so that it lives in SGPRs
    // (readfirstlane returns a signed int: go through uint32_t, or the low half would sign-extend)
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint64_t ub = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds)), "v"(voff), "s"(ub) : "memory", "m0");
}
__device__ __forceinline__ void phase_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int V> struct IntC { static constexpr int value = V; };

// ---------------------------------------------------------------------------
// First rows of a causal head, in the reference's own arithmetic.
//
// A query that sees only a handful of keys can produce outputs as large as
// the values themselves (|O| up to 4 and more at unit variance), where one
// fp16 ulp is the whole tolerance.  There the dominant error of the reference
// CPU verifier is its own rounding of every q*k and p*v product to the storage
// type (reference src/main.cu:193,259): it is off from the exact result by up
// to 3e-3 in those rows, and a kernel that accumulates exact products cannot
// land on the same side.  For the first kFaithfulRows rows of every head (at
// most that many visible keys under a causal mask) the workgroup therefore
// recomputes the result with exactly the reference's sequence: product
// rounded to the storage type, fp32 sums in index order, max-subtracted expf,
// fp32 normalisation, p rounded to the storage type (main.cu:189-263).  It is
// 32 x 32 scores and 32 x D outputs of scalar work per head.
// ---------------------------------------------------------------------------
constexpr int kFaithfulRows = 32;

// ---------------------------------------------------------------------------
// Dropout (role of reference src/flash_forward.h:248-265: after the softmax every P element is zeroed with
// probability p or multiplied by 1/(1-p); the row sums keep the undropped values).  The reference draws from
// per-thread curand states, which nothing can replay; here the decision is a pure function of
// (seed, batch*heads + head, query i, key j): one Philox4x32-10 block yields sixteen bytes for the sixteen keys
// j of a 32-key block that have the same (j / 4) % 2 -- exactly the keys of that block one lane of this kernel
// holds for its query -- and key j is kept iff its byte is >= the threshold (p in units of 1/256).
//   counter = (2 * (j / 32) + (j / 4) % 2,  i,  batch*heads + head,  0x44524F50),  key = (seed lo, seed hi)
//   byte index = 4 * ((j % 32) / 8) + j % 4, bytes numbered from the low byte of output word 0
// ---------------------------------------------------------------------------
struct DropWords { uint32_t w[4]; };
__device__ __forceinline__ DropWords dropout_words(uint32_t seed_lo, uint32_t seed_hi, uint32_t bh, uint32_t i, uint32_t group)
{
    uint32_t c0 = group, c1 = i, c2 = bh, c3 = 0x44524F50u, k0 = seed_lo, k1 = seed_hi;
#pragma unroll
    for (int round = 0; round < 10; ++round) {
        // (one 32 x 32 -> 64-bit multiply-add instruction per product instead of a high and a low multiply, each
        // of which runs at a quarter of the vector ALU's rate)
        const uint64_t p0 = (uint64_t)0xD2511F53u * (uint64_t)c0, p1 = (uint64_t)0xCD9E8D57u * (uint64_t)c2;
        const uint32_t h0 = (uint32_t)(p0 >> 32), l0 = (uint32_t)p0, h1 = (uint32_t)(p1 >> 32), l1 = (uint32_t)p1;
        // (the two three-way exclusive ors as one v_bitop3_b32 each, truth table 0x96; left to the compiler they
        // are two v_xor_b32 each)
        c0 = __builtin_amdgcn_bitop3_b32(h1, c1, k0, 0x96); c1 = l1; c2 = __builtin_amdgcn_bitop3_b32(h0, c3, k1, 0x96); c3 = l0;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    return DropWords{{c0, c1, c2, c3}};
}
__device__ __forceinline__ bool dropout_keep_byte(const DropWords &d, int r, uint32_t threshold)
{
    return ((d.w[r >> 2] >> (8 * (r & 3))) & 255u) >= threshold;
}

template <bool BF16> __device__ __forceinline__ float storage_to_f32(uint16_t h)
{
    if (BF16) return __builtin_bit_cast(float, (uint32_t)h << 16);
    return (float)__builtin_bit_cast(_Float16, h);
}
template <bool BF16> __device__ __forceinline__ uint16_t f32_to_storage(float x)
{
    if (BF16) return __builtin_bit_cast(uint16_t, (__bf16)x);
    return __builtin_bit_cast(uint16_t, (_Float16)x);
}
// Two storage-type products a.lo * b.lo and a.hi * b.hi of packed storage-type values, each rounded once to the
// storage type (round to nearest even) and widened to fp32: the reference's half x half -> half product
// (main.cu:193,259).  fp16: v_pk_mul_f16 rounds exactly so; the empty asm keeps the compiler from contracting
// the product with the addition that follows into one fused operation, which would skip the rounding.
// bf16: the fp32 product of two bf16 values is exact, then one rounding.
template <bool BF16> __device__ __forceinline__ f32x2 storage_product2(uint32_t a, uint32_t b)
{
    if (!BF16) {
        f16x2 pr = __builtin_bit_cast(f16x2, a) * __builtin_bit_cast(f16x2, b);
        uint32_t bits = __builtin_bit_cast(uint32_t, pr);
        asm volatile("" : "+v"(bits));
        pr = __builtin_bit_cast(f16x2, bits);
        return f32x2{(float)pr[0], (float)pr[1]};
    }
    const f32x2 exact = {__builtin_bit_cast(float, a << 16) * __builtin_bit_cast(float, b << 16),
                         __builtin_bit_cast(float, a & 0xffff0000u) * __builtin_bit_cast(float, b & 0xffff0000u)};
    const uint32_t r = __builtin_bit_cast(uint32_t, __builtin_convertvector(exact, bf16x2));
    return f32x2{__builtin_bit_cast(float, r << 16), __builtin_bit_cast(float, r & 0xffff0000u)};
}

// s0 += a.lo * b.lo and s1 += a.hi * b.hi with every product rounded to the storage type first (s0 and s1 may be
// the same sum: the low product is then added before the high one).  fp16: the rounded pair from v_pk_mul_f16 goes
// into the fp32 sums through v_fma_mix_f32 (x * 1.0 + sum with the half-precision operand widened on the way:
// the same bits as a conversion followed by an addition, in one instruction instead of two).
template <bool BF16> __device__ __forceinline__ void add_storage_products(uint32_t a, uint32_t b, float &s0, float &s1)
{
    if (!BF16) {
        f16x2 pr = __builtin_bit_cast(f16x2, a) * __builtin_bit_cast(f16x2, b);
        uint32_t bits = __builtin_bit_cast(uint32_t, pr);
        asm("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "+v"(s0) : "v"(bits));
        asm("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(s1) : "v"(bits));
        return;
    }
    const f32x2 pr = storage_product2<BF16>(a, b);
    s0 += pr[0];
    s1 += pr[1];
}

// Queries row0..row1-1 of a head (query i at key position i + pos_off, all positions below 32) against keys
// 0..31.  The 32 x D blocks of Q, K and V (the rows needed) are staged in LDS once (K with its 16-byte chunks
// XOR-swizzled by the row, so that 32 lanes reading one chunk of 32 different rows do not collide), everything
// else runs from there.  LDS use: 3 * 32 * D * 2 + 2 * 4096 + 128 bytes.
template <bool BF16, int D>
__device__ __forceinline__ void faithful_first_rows(const uint16_t *Qh, const uint16_t *Kh, const uint16_t *Vh, uint16_t *Oh,
                                    float *o32 /* null, or [rows][D] fp32 to write instead of Oh */,
                                    float *lse_h, int row0, int row1 /* queries row0..row1-1 */,
                                    int pos_off /* query i sits at key position i + pos_off */,
                                    int L, float scale, float slope,
                                    int q_rs, int k_rs, int v_rs, int o_rs /* row strides in elements */,
                                    uint32_t drop_threshold, float drop_scale, uint32_t seed_lo, uint32_t seed_hi, uint32_t bh,
                                    uint32_t lds /* LDS byte address of the work area */)
{
    constexpr int R = kFaithfulRows, CPR = D / 8;
    // (LDS-typed pointers: through generic ones every access would be a flat instruction)
    typedef __attribute__((address_space(3))) uint16_t lds_u16;
    typedef __attribute__((address_space(3))) float lds_f32;
    typedef __attribute__((address_space(3))) uint32_t lds_u32;
    typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
    lds_u16 *Qs = (lds_u16 *)(uintptr_t)lds, *Ks = Qs + R * D, *Vs = Ks + R * D;
    lds_f32 *sc = (lds_f32 *)(Vs + R * D), *ex = sc + R * R, *rsum = ex + R * R;
    lds_u32 *pbits = (lds_u32 *)ex;                         // after the softmax: p as two copies of its storage bits
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int nrows = row1 - row0;
    const int nkeys = row1 + pos_off;                       // keys 0..nkeys-1 are the ones any of these queries sees
    for (int idx = tid; idx < R * CPR; idx += nthr) {
        const int row = idx / CPR, c = idx % CPR;
        if (row >= row0 && row < row1)
            *(lds_u32x4 *)(Qs + row * D + 8 * c) = *reinterpret_cast<const u32x4 *>(Qh + (size_t)row * q_rs + 8 * c);
        if (row < nkeys) {
            *(lds_u32x4 *)(Ks + row * D + 8 * (c ^ (row & (CPR - 1)))) = *reinterpret_cast<const u32x4 *>(Kh + (size_t)row * k_rs + 8 * c);
            *(lds_u32x4 *)(Vs + row * D + 8 * c) = *reinterpret_cast<const u32x4 *>(Vh + (size_t)row * v_rs + 8 * c);
        }
    }
    __syncthreads();
    // scores (main.cu:189-197), masked entries -inf (main.cu:210-229); query i at position p sees keys p-L..p
    for (int idx = tid; idx < nrows * R; idx += nthr) {
        const int i = row0 + idx / R, j = idx % R, p = i + pos_off;
        float s = -INFINITY;
        if (j <= p && p - j <= L) {
            float sum = 0.0f;
            // (the operands are read four chunks at a time, ahead of the additions that have to wait for each other)
#pragma unroll
            for (int c0 = 0; c0 < CPR; c0 += 4) {
                u32x4 qa[4], kb[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    qa[c] = *(const lds_u32x4 *)(Qs + i * D + 8 * (c0 + c));
                    kb[c] = *(const lds_u32x4 *)(Ks + j * D + 8 * ((c0 + c) ^ (j & (CPR - 1))));
                }
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int w = 0; w < 4; ++w) {
                        add_storage_products<BF16>(qa[c][w], kb[c][w], sum, sum);
                    }
            }
            s = sum * scale;
            // ALiBi as the verifier applies it (main.cu:200-207): a rounded product, then a rounded difference
            if (slope != 0.0f) s = __fsub_rn(s, __fmul_rn(slope, (float)(p - j)));
        }
        sc[i * R + j] = s;
    }
    __syncthreads();
    // softmax of each row (main.cu:232-252).  The row maximum does not depend on the order it is taken in and
    // the exponentials are independent, so every thread does one element; only the row sum has to add in
    // index order, and one thread per row does that.
    for (int idx = tid; idx < nrows * R; idx += nthr) {
        const int i = row0 + idx / R, e = i * R + idx % R;
        const lds_f32 *row = sc + i * R;
        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < R; ++j) mx = fmaxf(mx, row[j]);
        ex[e] = sc[e] != -INFINITY ? expf(sc[e] - mx) : 0.0f;
    }
    __syncthreads();
    if (tid < nrows) {
        const int i = row0 + tid;
        const lds_f32 *row = ex + i * R;
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < R; ++j) sum += row[j];          // masked entries are +0: they change no bit of the sum
        rsum[i] = sum;
        if (lse_h != nullptr) {
            float mx = -INFINITY;
#pragma unroll
            for (int j = 0; j < R; ++j) mx = fmaxf(mx, sc[i * R + j]);
            lse_h[i] = mx + logf(sum);
        }
    }
    __syncthreads();
    // p rounded to the storage type (main.cu:259)
    for (int idx = tid; idx < nrows * R; idx += nthr) {
        const int i = row0 + idx / R, j = idx % R, e = i * R + j;
        float pj = 0.0f;
        if (sc[e] != -INFINITY) {
            pj = ex[e] / rsum[i];
            if (drop_threshold != 0u) {        // keys 0..31: one 32-key block, two Philox blocks per query
                const DropWords d = dropout_words(seed_lo, seed_hi, bh, (uint32_t)(i + pos_off), (uint32_t)((j >> 2) & 1));
                // (the word is picked with selects: indexed with a run-time value the four words would live in scratch memory)
                const int wi = j >> 3;
                const uint32_t word = wi == 0 ? d.w[0] : wi == 1 ? d.w[1] : wi == 2 ? d.w[2] : d.w[3];
                pj = ((word >> (8 * (j & 3))) & 255u) >= drop_threshold ? __fmul_rn(pj, drop_scale) : 0.0f;
            }
        }
        const uint32_t bits = f32_to_storage<BF16>(pj);
        pbits[e] = bits | (bits << 16);         // (each thread overwrites only the element it has just read)
    }
    __syncthreads();
    // weighted sum (main.cu:255-263), keys in ascending order; masked keys have p = 0 and add nothing.  A thread
    // owns two neighbouring output elements of one row.
    for (int idx = tid; idx < nrows * (D / 2); idx += nthr) {
        const int i = row0 + idx / (D / 2), t2 = idx % (D / 2), p = i + pos_off;
        const int lo = p - L > 0 ? p - L : 0;
        float s0 = 0.0f, s1 = 0.0f;
        // (all operands are read first, with a fixed trip count, and the additions follow in key order under a
        // predicate: read one by one inside a loop from lo to p, every step waited for its own LDS round trip,
        // 85 ns per key)
        uint32_t pw[R], vw[R];
#pragma unroll
        for (int j = 0; j < R; ++j) {
            pw[j] = pbits[i * R + j];
            vw[j] = *(const lds_u32 *)(Vs + j * D + 2 * t2);        // (rows past the last key hold stale bytes: never used)
        }
#pragma unroll
        for (int j = 0; j < R; ++j) {
            if (j >= lo && j <= p) {
                add_storage_products<BF16>(pw[j], vw[j], s0, s1);
            }
        }
        const uint32_t packed = Num<BF16>::pack2(s0, s1);
        if (o32 != nullptr) {
            o32[(size_t)i * D + 2 * t2] = storage_to_f32<BF16>((uint16_t)(packed & 0xffffu));
            o32[(size_t)i * D + 2 * t2 + 1] = storage_to_f32<BF16>((uint16_t)(packed >> 16));
        } else {
            *reinterpret_cast<uint32_t *>(Oh + (size_t)i * o_rs + 2 * t2) = packed;
        }
    }
    __syncthreads();
}

// ---------------------------------------------------------------------------
// The kernel.  NW waves per workgroup, 32 query rows per wave, NST LDS stages
// per tensor.  Every wave runs ONE instruction stream per key tile; tiles are
// issued NST-1 iterations before their first use; one workgroup barrier per
// tile.  Two waves per SIMD (at most 256 registers each).
// ---------------------------------------------------------------------------
template <int N> __device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }

template <bool BF16, int D, bool MASKED, bool ALIBI, bool GENERAL, bool DROPOUT, int NW, int NST, bool STRIDED = false, int NSTV = NST>
__global__ void __launch_bounds__(NW * 64, 2) fa_fwd_pipelined(const FaKernelArgs a)
{
    constexpr int WR = 32;                        // query rows per wave
    constexpr int BR = WR * NW;                   // query rows per workgroup
    constexpr int CPR = D / 8;
    constexpr int ROWB = D * 2;
    constexpr int TILEB = kBlockKeys * ROWB;
    constexpr int INSTR = TILEB / 1024;
    constexpr int IPW = INSTR / NW;               // direct-to-LDS instructions per wave per tile
    constexpr int KS = D / 16;
    constexpr int DB = D / 32;
    constexpr int NPV = 4 * DB;                   // V^T fragments per tile: (16-key slice, head-dim block)
    constexpr int NQK = 2 * KS;                   // K fragments per tile: (head-dim slice, 32-key block)
    constexpr int NF = NPV + NQK;                 // every fragment feeds one matrix instruction
    constexpr int PD = 6;                         // LDS reads run this many fragments ahead
    constexpr int LA = NST - 1;                   // K tiles are requested LA iterations before their first use
    constexpr int LAV = NSTV - 1;                 // V tiles likewise (NSTV V stages: as many as K stages, or one fewer)
    constexpr int STAGES = NST + NSTV;
    // (the first-rows path works in LDS behind the K stages that the requests for the next item fill)
    static_assert(GENERAL || LA * TILEB + NW * 32 * ROWB <= STAGES * TILEB, "the epilogue's row blocks do not fit behind the requested stages");
    static_assert(NST <= 3 && LA * TILEB + 3 * kFaithfulRows * D * 2 + 2 * 4096 + 128 <= STAGES * TILEB, "first-rows path does not fit behind the requested stages");
    static_assert(NSTV == NST || (NSTV == NST - 1 && NSTV >= 2), "V stages: as many as K stages, or one fewer");
    constexpr uint32_t LDS_V = NST * TILEB;       // K stages first, then V stages
    static_assert(INSTR % NW == 0, "tile must divide over the waves");
    static_assert(NST >= 2 && NST * TILEB <= 65536, "stage offsets must fit the 16-bit LDS immediate");
    typedef Num<BF16> N;

    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int half = lane >> 5, l32 = lane & 31, l16 = lane & 15;

    // Work items.  Without a queue the grid is static: one workgroup per item (a single pass), or a resident
    // grid that walks the longest-first list as a snake (pass 0 forwards, pass 1 backwards, ...), pairing
    // long items with short ones.  With a queue, a resident grid takes items dynamically: a workgroup on XCD x
    // takes list positions x, x+8, x+16, ... from that XCD's counter, so a head stays on one XCD's L2 and a
    // workgroup that finishes early simply takes the next item -- the hardware dispatcher's longest-first
    // greedy schedule without its workgroup launch gaps (about 10 us per item on this chip).
    const int G = (int)gridDim.x;
    unsigned xcd = 0;
    if (a.queue != nullptr) {
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcd));
        xcd &= 7u;
    }
    // next_slot broadcasts the list position a queue-scheduled workgroup has taken
    volatile __attribute__((address_space(3))) unsigned *next_slot =
        (volatile __attribute__((address_space(3))) unsigned *)(uintptr_t)(lds0 + STAGES * TILEB - 64);
    constexpr unsigned kNoTicket = 0xffffffffu;
    // The work item of pass `pass_no` of this workgroup, or -1 when its work is done (list positions fit 31
    // bits, the host checks that).  Queue schedule: `ticket` is the value of the own XCD's counter when thread 0
    // has fetched it ahead of time, or kNoTicket.
    auto take_item = [&](int pass_no, unsigned ticket) __attribute__((always_inline)) -> int {
        if (a.queue == nullptr) {
            const long long base = (long long)pass_no * G;
            const long long it = base + ((pass_no & 1) ? G - 1 - (int)blockIdx.x : (int)blockIdx.x);
            return it < a.n_items ? (int)it : -1;     // (an odd pass may leave this workgroup out; the next is empty then)
        }
        if (tid == 0) {
            // own XCD's list first; when that is exhausted, help the others (this also makes the result
            // independent of how the hardware spreads the workgroups over the XCDs)
            // (When the own list is exhausted, all eight counters are read in one round trip before any is
            // updated: a workgroup that finds nothing left then pays for one read instead of eight updates in
            // a row, on counters that every other leaving workgroup updates at the same time.)
            unsigned found = 0xffffffffu;
            if (ticket == kNoTicket) ticket = atomicAdd(&a.queue[xcd], 1u);
            const long long own = (long long)ticket * 8 + xcd;
            if (own < a.n_items) found = (unsigned)own;
            while (found == 0xffffffffu) {
                unsigned cnt[8];
#pragma unroll
                for (unsigned xo = 1; xo < 8u; ++xo)
                    cnt[xo] = __hip_atomic_load(&a.queue[(xcd + xo) & 7u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                unsigned pick = 8u;
#pragma unroll
                for (unsigned xo = 7; xo >= 1u; --xo)
                    if ((long long)cnt[xo] * 8 + ((xcd + xo) & 7u) < a.n_items) pick = xo;
                if (pick == 8u) break;
                const unsigned xq = (xcd + pick) & 7u;
                const long long cand = (long long)atomicAdd(&a.queue[xq], 1u) * 8 + xq;
                if (cand < a.n_items) found = (unsigned)cand;
            }
            *next_slot = found;
        }
        __syncthreads();
        // uniform by construction: say so, or everything derived from the item lives in vector registers
        const int taken = __builtin_amdgcn_readfirstlane((int)*next_slot);
        __syncthreads();
        return taken;
    };
    // The next work item is taken before the epilogue of the current one, and (contiguous layout) its Q^T
    // fragments and first K tiles are requested there: the 3-5 us their first bytes take to arrive from HBM lie
    // behind the epilogue instead of in front of the next tile loop.
    u32x4 qf[KS];
    bool next_requested = false;
    int item = take_item(0, kNoTicket);
    for (int pass = 0; item >= 0; ++pass) {
    int bh, qblock;
    // (GENERAL with key splits: consecutive list positions are the splits of one (head, query block))
    const int n_splits = GENERAL ? a.n_splits : 1;
    // (list positions fit 31 bits, the host checks that: 32-bit divisions)
    const unsigned head_item = n_splits > 1 ? (unsigned)item / (unsigned)n_splits : (unsigned)item;
    const int split = n_splits > 1 ? (int)((unsigned)item - head_item * (unsigned)n_splits) : 0;
    // (GENERAL, packed groups: an item is a (batch, K/V head); its rows are the queries of all query heads
    // of that K/V head, head after head -- few queries against long keys read K and V once per group)
    const int pack = GENERAL ? a.pack : 1;
    fa_item_decode((long long)head_item, pack > 1 ? a.BH / pack : a.BH, a.n_qblocks, a.descending, &bh, &qblock);
    const int S = a.S;
    // GENERAL: Sk keys; query i sits at key position i + pos_off (the queries are the last S positions), which
    // is what masks, the ALiBi distance and the dropout decision see.
    const int Sk = GENERAL ? a.Sk : S;
    const int pos_off = GENERAL ? a.Sk - a.S : 0;
    // Contiguous [B,H,S,D] tensors, one K/V head per query head, S a multiple of 128: everything below is
    // compile-time.  GENERAL: any strides (in elements, head dimension contiguous), query heads sharing K/V
    // heads in groups of H/Hk, any S (rows past the end are read from row S-1 and never stored, keys past the
    // end are masked like any other masked key).
    const uint16_t *Qh, *Kh, *Vh;
    uint16_t *Oh;
    if (GENERAL) {
        // Query heads that share a K/V head: the list walks the K/V heads fastest (list position -> XCD is
        // round robin, so with a multiple of eight K/V heads all query heads of one K/V head run on the XCD
        // whose L2 holds that head's K and V) and the members of a group slowest.
        int bi, hk, hi;
        if (pack > 1) {             // bh counts (batch, K/V head); hi is the first query head of the group
            bi = bh / a.Hk; hk = bh - bi * a.Hk; hi = hk * pack;
        } else {
            const int r = bh % a.H, group = a.H / a.Hk;
            bi = bh / a.H;
            hk = group > 1 ? r % a.Hk : r;
            hi = group > 1 ? hk * group + r / a.Hk : r;
        }
        bh = bi * a.H + hi;         // from here on the real head index (logsumexp, ALiBi slope, dropout)
        Qh = a.Q + (size_t)bi * a.q_bs + (size_t)hi * a.q_hs;
        Kh = a.K + (size_t)bi * a.k_bs + (size_t)hk * a.k_hs;
        Vh = a.V + (size_t)bi * a.v_bs + (size_t)hk * a.v_hs;
        Oh = a.O + (size_t)bi * a.o_bs + (size_t)hi * a.o_hs;
    } else {
        if (STRIDED) {
        // (grouped K/V heads as in the general kernels: the list walks the K/V heads fastest, so that the query
        // heads of one K/V head run on the XCD whose L2 holds its K and V)
        int hi, hk;
        const int bi = fa_strided_heads(bh, a.H, a.Hk, &hi, &hk);
        bh = bi * a.H + hi;         // from here on the real head index (logsumexp, ALiBi slope)
        Qh = a.Q + (size_t)bi * a.q_bs + (size_t)hi * a.q_hs;
        Kh = a.K + (size_t)bi * a.k_bs + (size_t)hk * a.k_hs;
        Vh = a.V + (size_t)bi * a.v_bs + (size_t)hk * a.v_hs;
        Oh = a.O + (size_t)bi * a.o_bs + (size_t)hi * a.o_hs;
        } else {
        const size_t head_off = (size_t)bh * S * D;
        Qh = a.Q + head_off; Kh = a.K + head_off; Vh = a.V + head_off;
        Oh = a.O + head_off;
        }
    }
    const int q_rs = (GENERAL || STRIDED) ? a.q_rs : D, k_rs = (GENERAL || STRIDED) ? a.k_rs : D, v_rs = (GENERAL || STRIDED) ? a.v_rs : D,
              o_rs = (GENERAL || STRIDED) ? a.o_rs : D;

    const int q0 = qblock * BR;
    const int qw = q0 + wave * WR;          // first query row of this wave
    const int my_q = qw + l32;              // query row on this lane
    const int n_rows = pack * S;            // rows of this (head | packed group)
    const bool wave_live = qw < n_rows;     // (not GENERAL: S is a multiple of 128, a live wave has all its rows)
    // This lane's row: the query position inside its head, the head relative to `bh`, whether the row exists (a
    // row that does not exist computes on a copy of the last row and stores nothing).
    const bool row_ok = !GENERAL || my_q < n_rows;
    const int row_clamped = row_ok ? my_q : n_rows - 1;
    const int row_head = pack > 1 ? row_clamped / S : 0;
    const int row_pos = pack > 1 ? row_clamped - row_head * S : row_clamped;
    // the query positions this wave covers, for tile ranges and tile classes: its 32 rows when they lie in one
    // head, every position when they wrap from one head of a packed group into the next
    int wave_pos0 = qw, wave_npos = WR, block_pos0 = q0;
    if (pack > 1) {
        const int last = qw + WR - 1 < n_rows - 1 ? qw + WR - 1 : n_rows - 1;
        const bool one_head = wave_live && qw / S == last / S;
        wave_pos0 = one_head ? qw % S : 0;
        wave_npos = one_head ? last - qw + 1 : S;
        block_pos0 = 0;
    }

    // Q^T fragments: B operand, lane = (query l32, head-dim slice 8*half..+7 of each 16)
    if (!next_requested) {
#pragma unroll
        for (int s = 0; s < KS; ++s)
            qf[s] = wave_live ? *reinterpret_cast<const u32x4 *>(
                                    Qh + (GENERAL ? (size_t)row_head * a.q_hs : 0) + (size_t)row_pos * q_rs + 16 * s + 8 * half)
                              : u32x4{0, 0, 0, 0};
    }

    const int rows_in_block = pack > 1 ? S : S - q0 < BR ? S - q0 : BR;
    int t0, t1;                 // key tiles visited by the workgroup
    fa_tile_range(Sk, kBlockKeys, a.L, a.R, block_pos0 + pos_off, rows_in_block, &t0, &t1);
    int my_lo = 1, my_hi = 0;   // key tiles with at least one visible pair for this wave (contiguous)
    if (wave_live) fa_tile_range(Sk, kBlockKeys, a.L, a.R, wave_pos0 + pos_off, wave_npos, &my_lo, &my_hi);
    if (n_splits > 1) {         // this item's share of the key tiles; may leave nothing
        const int s_lo = split * a.tiles_per_split, s_hi = s_lo + a.tiles_per_split - 1;
        t0 = t0 > s_lo ? t0 : s_lo;
        t1 = t1 < s_hi ? t1 : s_hi;
        my_lo = my_lo > s_lo ? my_lo : s_lo;
        my_hi = my_hi < s_hi ? my_hi : s_hi;
    }
    const bool any_tile = !GENERAL || t0 <= t1;

    // per-lane LDS read addresses for stage 0; stage, key block and key slice are immediates
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
    // direct global -> LDS tile loads: wave w issues instructions w, w+NW, ... of the tile; instruction n
    // fills LDS bytes [n*1024, n*1024+1024) linearly, lane l supplying the swizzled source chunk.
    uint32_t gk[IPW], gv[IPW];
#pragma unroll
    for (int i = 0; i < IPW; ++i) {
        const int P = (i * NW + wave) * 64 + lane, row = P / CPR, pos = P % CPR;
        gk[i] = (uint32_t)(row * (k_rs * 2) + ((pos ^ k_swz<CPR>(row)) << 4));
        gv[i] = (uint32_t)(row * (v_rs * 2) + ((pos ^ v_swz<CPR>(row)) << 4));
    }
    // (GENERAL: the rows of the last tile that lie past the end of the sequence are fetched from row S-1;
    // they land in their own LDS rows and are masked)
    auto ragged_source = [&](int tile, int i, int rs, bool is_k) __attribute__((always_inline)) {
        const int P = (i * NW + wave) * 64 + lane, row = P / CPR, pos = P % CPR;
        const int last = Sk - 1 - tile * kBlockKeys, src_row = row < last ? row : last;
        return (uint32_t)(src_row * (rs * 2) + ((pos ^ (is_k ? k_swz<CPR>(row) : v_swz<CPR>(row))) << 4));
    };
    auto issue_k_from = [&](const uint16_t *k_head, int tile, int stage) __attribute__((always_inline)) {
        const char *src = reinterpret_cast<const char *>(k_head) + (size_t)tile * (kBlockKeys * 2) * k_rs;
        const bool ragged = GENERAL && (tile + 1) * kBlockKeys > Sk;
#pragma unroll
        for (int i = 0; i < IPW; ++i)
            dma_16(src, ragged ? ragged_source(tile, i, k_rs, true) : gk[i], lds0 + stage * TILEB + (i * NW + wave) * 1024);
    };
    auto issue_k = [&](int tile, int stage) __attribute__((always_inline)) { issue_k_from(Kh, tile, stage); };
    auto issue_v_from = [&](const uint16_t *v_head, int tile, int stage) __attribute__((always_inline)) {
        const char *src = reinterpret_cast<const char *>(v_head) + (size_t)tile * (kBlockKeys * 2) * v_rs;
        const bool ragged = GENERAL && (tile + 1) * kBlockKeys > Sk;
#pragma unroll
        for (int i = 0; i < IPW; ++i)
            dma_16(src, ragged ? ragged_source(tile, i, v_rs, false) : gv[i], lds0 + LDS_V + stage * TILEB + (i * NW + wave) * 1024);
    };
    auto issue_v = [&](int tile, int stage) __attribute__((always_inline)) { issue_v_from(Vh, tile, stage); };
    // skip / edge / free classification of a key tile for this wave (GENERAL: a tile that reaches past the
    // end of the sequence is an edge tile)
    auto tile_class = [&](int tile) __attribute__((always_inline)) {
        int cls = fa_tile_class(kBlockKeys, a.L, a.R, wave_pos0 + pos_off, wave_npos, tile);
        if (GENERAL && cls == 2 && (tile + 1) * kBlockKeys > Sk) cls = 1;
        return cls;
    };

    f32x16 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] = 0.0f;
    // reference point of the exponentials (raw score units), row-sum halves.  (The reference point starts from a
    // finite value far below every score: the first finite row maximum moves it, with a factor exp2(-huge) = 0
    // for the empty accumulators, and no place needs a test for -inf.)
    float m_run = kNoReference, l_a = 0.0f, l_b = 0.0f;
    // The tile scores stay raw dot products and the softmax scale is folded into the exponent (exp2(s*c - m*c)).
    // ALiBi (mask.h:21-26 subtracts slope*|i-j| from the scaled score) enters through the matrix instruction's
    // accumulator: the first product of a key block starts from -(slope/scale)*|i-j| instead of from zero, two
    // vector instructions per score element in front of that instruction, and everything behind it is the code
    // of the kernels without ALiBi.  (Rewriting the finished tile, s*c - slope*log2(e)*|i-j|, took three per
    // element in the serial phase of the iteration.)
    const float c = a.scale_log2e;
    const float cs = c;
    // (one slope per head: per lane when the rows of a wave belong to several heads of a packed group)
    const float slope = ALIBI ? a.alibi[bh % a.H + (GENERAL ? row_head : 0)] : 0.0f;
    const float neg_slope_raw = ALIBI ? -slope / a.scale : 0.0f;        // per key of distance, in raw score units
    const float thresh = kRescaleLog2 / cs;
    uint32_t pk[16];            // P of the tile whose PV comes next: [0..7] keys 0..31, [8..15] keys 32..63
    f32x16 sx[2];               // S^T of the tile whose softmax comes next: [key block 0 / 1]

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
        const int q = row_pos + pos_off;
        // last visible key of this query (GENERAL: the sequence may end inside the tile)
        const int j_hi = (GENERAL && q + a.R > Sk - 1) ? Sk - 1 : q + a.R;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int j0 = kb0 + 8 * (r >> 2) + (r & 3);
            const int j1 = j0 + 32;
            if (j0 > j_hi || j0 < q - a.L) sx[0][r] = -INFINITY;
            if (j1 > j_hi || j1 < q - a.L) sx[1][r] = -INFINITY;
        }
    };
    // the initial accumulator of key block `blk` of `tile`
    auto alibi_start = [&](int blk, int tile) __attribute__((always_inline)) {
        // signed distance of this lane's query to the lane's first key of the block: exact in fp32
        const float base = (float)(row_pos + pos_off - (tile * kBlockKeys + 32 * blk + 4 * half));
        f32x16 v;
        if (MASKED && a.R == 0) {
            // no visible key lies behind its query: the distance is base - k without the absolute value (the
            // elements for which that is wrong are masked), one fused multiply-add with the key offset as a literal
            const float at_base = base * neg_slope_raw;
#pragma unroll
            for (int r = 0; r < 16; ++r) v[r] = __builtin_fmaf((float)(8 * (r >> 2) + (r & 3)), -neg_slope_raw, at_base);
        } else {
#pragma unroll
            for (int r = 0; r < 16; ++r) v[r] = __builtin_fabsf(base - (float)(8 * (r >> 2) + (r & 3))) * neg_slope_raw;
        }
        return v;
    };
    auto row_max = [&]() __attribute__((always_inline)) {
        float mx = max_plain(sx[0][0], sx[1][0]);
#pragma unroll
        for (int r = 1; r < 16; ++r) mx = fmaxf(fmaxf(mx, sx[0][r]), sx[1][r]);
        return max_of_halves(mx);
    };
    // the decision to move the reference point; returns the factor by which everything accumulated so far has to
    // be multiplied (1 when the reference point stays)
    auto new_reference = [&](float mx, bool &moved) __attribute__((always_inline)) {
        float alpha = 1.0f;
        const bool grow = mx > m_run + thresh;      // (from kNoReference every finite maximum grows)
        moved = __builtin_amdgcn_ballot_w64(grow) != 0;
        if (moved) {
            const float m_new = grow ? mx : m_run;
            alpha = __builtin_amdgcn_exp2f((m_run - m_new) * cs);
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
    auto p_operand = [&](int t2) __attribute__((always_inline)) {
        return u32x4{pk[4 * t2], pk[4 * t2 + 1], pk[4 * t2 + 2], pk[4 * t2 + 3]};
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
            o[db] = N::mfma(fr[n], p_operand(t2), o[db]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto qk_plain = [&](int kstage, int tile) __attribute__((always_inline)) {
        const uint32_t ks = kstage * TILEB;
        u32x4 fr[NQK];
        fr[0] = read_k(ks, 0);
        fr[1] = read_k(ks, 1);
#pragma unroll
        for (int r = 0; r < 16; ++r) { sx[0][r] = 0.0f; sx[1][r] = 0.0f; }
        if (ALIBI) { sx[0] = alibi_start(0, tile); sx[1] = alibi_start(1, tile); }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int n = 0; n < NQK; ++n) {
            if (n + 2 < NQK) fr[n + 2] = read_k(ks, n + 2);
            sx[n & 1] = N::mfma(fr[n], qf[n >> 1], sx[n & 1]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // dropout decisions of the tile whose exponentials come next: per key block the sixteen bytes for this
    // lane's sixteen keys
    DropWords dw[2];
    auto draw_dropout = [&](int tile) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
            dw[kb] = dropout_words(a.seed_lo, a.seed_hi, (uint32_t)(bh + (GENERAL ? row_head : 0)),
                                   (uint32_t)(row_pos + pos_off), (uint32_t)(2 * (2 * tile + kb) + half));
    };
    auto dropped = [&](float e, int kb, int r) __attribute__((always_inline)) {
        if (!DROPOUT) return e;
        // (a kept probability's factor 1 / (1 - p) is the same for all of them: it multiplies the row once, in the
        // epilogue, instead of 32 elements per lane and tile here)
        return dropout_keep_byte(dw[kb], r, a.drop_threshold) ? e : 0.0f;
    };
    auto softmax_plain = [&](int tile) __attribute__((always_inline)) {
        if (DROPOUT) draw_dropout(tile);
        if (MASKED && tile_class(tile) == 1) apply_mask(tile);
        bool moved;
        const float alpha = new_reference(row_max(), moved);
        if (moved) scale_o(alpha);
        const float mc = m_run * cs;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sx[0][2 * i], cs, -mc));
            const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sx[0][2 * i + 1], cs, -mc));
            const float e2 = __builtin_amdgcn_exp2f(__builtin_fmaf(sx[1][2 * i], cs, -mc));
            const float e3 = __builtin_amdgcn_exp2f(__builtin_fmaf(sx[1][2 * i + 1], cs, -mc));
            l_a += e0; l_b += e1; l_a += e2; l_b += e3;
            pk[i] = N::pack2(dropped(e0, 0, 2 * i), dropped(e1, 0, 2 * i + 1));
            pk[8 + i] = N::pack2(dropped(e2, 1, 2 * i), dropped(e3, 1, 2 * i + 1));
        }
    };

    // ---- the steady-state iteration: PV(tile-1) from V stage VST, softmax(tile), QK(tile+1) from K stage KST
    auto steady = [&](auto KST, auto VST, int vstage_rt, int tile) __attribute__((always_inline)) {
        constexpr uint32_t ks = decltype(KST)::value * TILEB;
        // (with as many V stages as K stages the V stage is a compile-time value like the K stage; with one fewer
        // the two cycle with different periods, and the V stage is a run-time offset added to the lanes' addresses)
        const uint32_t vs = NSTV == NST ? decltype(VST)::value * TILEB : (uint32_t)vstage_rt * TILEB;
        u32x4 fr[NF];                              // operand fragments, in the order they are consumed
        auto fetch = [&](int n) __attribute__((always_inline)) {
            if (n < NPV) fr[n] = read_v(vs, n);
            else fr[n] = read_k(ks, n - NPV);
        };
#pragma unroll
        for (int n = 0; n < PD; ++n) fetch(n);
        // (Dropout: the tile's two Philox blocks are drawn here, in one piece.  Spread over the first ten matrix
        // instructions, two rounds each, they measured 1-5 % slower: with dropout the iteration is bound by the
        // vector ALU, not by the matrix pipe it would be hiding behind.)
        if (DROPOUT) draw_dropout(tile);
        // the fragments are in flight; the row maxima need no matrix instruction and cover their latency
        if (MASKED && tile_class(tile) == 1) apply_mask(tile);
        // The row maximum rides along with the first MAXG matrix instructions of PV(tile-1), which do not depend on
        // it (a quarter of the 32 scores per lane each); the reference point moves behind the last of them, without
        // a branch: a factor of exactly 1 where it stays.  The exponentials follow over the remaining instructions.
        constexpr int MAXG = FA_ROW_MAX_SLOTS;
        static_assert(MAXG == 0 || (16 % MAXG == 0 && MAXG < NPV), "row-maximum slots");
        bool moved = false;
        float alpha = 1.0f, nmc = 0.0f, mx = 0.0f;
        if (MAXG == 0) {
            alpha = new_reference(row_max(), moved);
            nmc = -m_run * cs;
        }
        uint32_t pn[16];                           // P(tile), becomes pk at the end
        f32x16 nx[2];                              // S^T(tile+1)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < NF; ++g) {
            if (g + PD < NF) fetch(g + PD);
            if (g < NPV) {
                const int t2 = g / DB, db = g % DB;
                o[db] = N::mfma(fr[g], p_operand(t2), o[db]);
            } else {
                const int n = g - NPV;
                const f32x16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
                nx[n & 1] = N::mfma(fr[g], qf[n >> 1], n >= 2 ? nx[n & 1] : ALIBI ? alibi_start(n & 1, tile + 1) : zero);
            }
            if (g < MAXG) {
                constexpr int PER = MAXG > 0 ? 16 / MAXG : 16;
                if (g == 0) mx = max_plain(sx[0][0], sx[1][0]);
                asm volatile("" : "+v"(mx));
#pragma unroll
                for (int r = g * PER + (g == 0 ? 1 : 0); r < (g + 1) * PER; ++r) mx = fmaxf(fmaxf(mx, sx[0][r]), sx[1][r]);
                if (g == MAXG - 1) {
                    mx = max_of_halves(mx);
                    const bool grow = mx > m_run + thresh;      // (from kNoReference every finite maximum grows)
                    moved = __builtin_amdgcn_ballot_w64(grow) != 0;
                    const float m_new = grow ? mx : m_run;
                    alpha = __builtin_amdgcn_exp2f((m_run - m_new) * cs);
                    l_a *= alpha;
                    l_b *= alpha;
                    m_run = m_new;
                    nmc = -m_new * cs;
                    asm volatile("" : "+v"(nmc), "+v"(l_a), "+v"(l_b));
                } else {
                    asm volatile("" : "+v"(mx));
                }
                __builtin_amdgcn_sched_barrier(0);
                continue;
            }
            // softmax work riding along: the 16 element pairs of this tile spread over the matrix instructions
            constexpr int PAIRS = 16;
            const int p_begin = ((g - MAXG) * PAIRS) / (NF - MAXG), p_end = ((g - MAXG + 1) * PAIRS) / (NF - MAXG);
#pragma unroll
            for (int e = p_begin; e < p_end; ++e) {
                // pair e: elements (2e, 2e+1) of key block 0 for e < 8, of key block 1 for e >= 8.  The two empty
                // asm statements pin the arithmetic between the surrounding matrix instructions (without them the
                // compiler sinks all of it to the end of the iteration); the first goes through the subtrahend,
                // which stays in one register, so it costs no move.
                const float x0 = e < 8 ? sx[0][2 * e] : sx[1][2 * (e - 8)];
                const float x1 = e < 8 ? sx[0][2 * e + 1] : sx[1][2 * (e - 8) + 1];
                asm volatile("" : "+v"(nmc));
                const float e0 = __builtin_amdgcn_exp2f(__builtin_fmaf(x0, c, nmc));
                const float e1 = __builtin_amdgcn_exp2f(__builtin_fmaf(x1, c, nmc));
                l_a += e0;
                l_b += e1;
                uint32_t packed = N::pack2(dropped(e0, e >> 3, 2 * (e & 7)), dropped(e1, e >> 3, 2 * (e & 7) + 1));
                asm volatile("" : "+v"(packed), "+v"(l_a), "+v"(l_b));
                pn[e] = packed;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (moved) scale_o(alpha);                 // rare; PV(tile-1) has been issued in full by now
#pragma unroll
        for (int i = 0; i < 16; ++i) pk[i] = pn[i];
        sx[0] = nx[0];
        sx[1] = nx[1];
    };

    unsigned ticket_ahead = kNoTicket;      // thread 0 only
    if (any_tile) {             // (GENERAL: a split, or a block of rows that sees no key, may have no tile at all)
    // ---- prologue: K(t0) .. K(t0+LA-1) requested before the first iteration (iteration i requests K(i+1+LA) and
    // V(i-1+LAV), and the first one is i = t0 - 1)
    if (!next_requested) {
        issue_k(t0, 0);
        if (LA > 1 && t0 + 1 <= t1) issue_k(t0 + 1, 1);
    }
    next_requested = false;
    wait_vm<0>();
    // Q has landed too (vmcnt is 0).  Touching the fragments here lets the compiler see that, so that it places
    // no vmcnt wait of its own inside the loop, where it would also wait for the asynchronous tile loads.
#pragma unroll
    for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]));
    phase_barrier();

    // Iteration j (tile i = t0 - 1 + j) does PV(i-1), softmax(i), QK(i+1).  Tile t0 + r lives in stage r % NST of
    // K and r % NSTV of V, so the iteration reads K stage j % NST and V stage (j - 2) % NSTV; it issues the loads of
    // K(i+1+LA) and V(i-1+LAV), which overwrite tiles whose last readers ran one iteration ago.
    // Every wave executes every iteration (one barrier each); a wave whose own tile range does not cover all
    // three pieces runs the plain pieces it has, the others run the interleaved body.  The two kinds live in
    // separate loops: merging them under one branch makes the register allocator spill.
    auto finish_iteration = [&](bool more_k, bool more_v, bool past_last_request) __attribute__((always_inline)) {
        // What the next iteration reads must have landed.  With LA = LAV = 2 that was requested one iteration ago,
        // so this iteration's requests may stay in flight (vmcnt counts requests, so this only holds while the
        // iteration made all of its 2 * IPW requests).  With LAV = 1 (one V stage fewer) the next iteration reads
        // the V tile requested in this one: V is requested in front of K, and only K's requests stay in flight.
        if (NSTV == NST && NST >= 3 && more_k && more_v) wait_vm<2 * IPW>();
        else if (NSTV < NST && more_k) wait_vm<IPW>();
        // (the last iterations of an item, those past the request for V(t1), request nothing, and the one before
        // them has waited for everything: they do not wait, so that the counter fetched there for the next
        // item stays in flight)
        else if (!past_last_request) wait_vm<0>();
        phase_barrier();
    };
#ifdef FA_CHECK_RING
    // Checking build: the invariants of the LDS ring, asserted by every wave in every iteration.  In front of the
    // iteration's work and again behind it (in front of the barrier that releases the stages), K stage `kstage` must
    // hold key tile i + 1 and V stage `vstage` key tile i - 1: each lane compares sixteen bytes of both stages with
    // the same bytes read from global memory.  A tile that has not landed when it is read (a wait that counts too
    // few requests, a missing barrier) or that is overwritten while others still read it (a request issued a stage
    // too early) shows up as a mismatch; nothing traps, the counters are read by the host afterwards.
    auto ring_check = [&](int i, int kstage, int vstage, int salt) __attribute__((always_inline)) {
        const int row = lane, chunk = (wave + salt) % CPR;          // one 16-byte chunk per lane
        unsigned long long checked = 0, bad = 0;
        for (int which = 0; which < 2; ++which) {
            const int tile = which == 0 ? i + 1 : i - 1;
            if (tile < t0 || tile > t1) continue;
            const int key = tile * kBlockKeys + row;
            if (key >= Sk) continue;                                 // (GENERAL: rows past the end hold copies of the last row)
            const int swz = which == 0 ? k_swz<CPR>(row) : v_swz<CPR>(row);
            const uint32_t addr = lds0 + (which == 0 ? 0u : LDS_V) + (uint32_t)((which == 0 ? kstage : vstage) * TILEB + row * ROWB + ((chunk ^ swz) << 4));
            const u32x4 in_lds = lds_read_b128(addr);
            const uint16_t *src = (which == 0 ? Kh + (size_t)key * k_rs : Vh + (size_t)key * v_rs) + 8 * chunk;
            const u32x4 in_mem = *reinterpret_cast<const u32x4 *>(src);
            ++checked;
            if (in_lds[0] != in_mem[0] || in_lds[1] != in_mem[1] || in_lds[2] != in_mem[2] || in_lds[3] != in_mem[3]) ++bad;
        }
        // (the compiler's wait for the global loads above is a wait for every request in flight: it can only hide a
        // violation that would have happened after this point, never produce one)
        if (a.ring_check != nullptr) {
            if (checked) atomicAdd(&a.ring_check[0], checked);
            if (bad) atomicAdd(&a.ring_check[1], bad);
        }
    };
#define FA_RING_CHECK(i, ks, vs, salt) ring_check(i, ks, vs, salt)
#else
#define FA_RING_CHECK(i, ks, vs, salt) do { } while (0)
#endif
    // V stage read by the iteration with K stage j3 and run-time V counter jv (= (j - 2) mod NSTV), and the V stage
    // it requests into (the one read one iteration ago)
    auto generic_iteration = [&](int i, int j3, int jv) __attribute__((always_inline)) {
        const int tk = i + 1 + LA, tv = i - 1 + LAV;
        const bool more_k = tk <= t1, more_v = tv >= t0 && tv <= t1;
        const int jm1 = j3 == 0 ? NST - 1 : j3 - 1, jm2 = jm1 == 0 ? NST - 1 : jm1 - 1, jm3 = jm2 == 0 ? NST - 1 : jm2 - 1;
        const int v_read = NSTV == NST ? jm2 : jv, v_fill = NSTV == NST ? jm3 : (jv == 0 ? NSTV - 1 : jv - 1);
        if (NSTV < NST && more_v) issue_v(tv, v_fill);     // (in front of K: see finish_iteration)
        if (more_k) issue_k(tk, jm1);              // (j + LA) % NST == (j - 1) % NST
        if (NSTV == NST && more_v) issue_v(tv, v_fill);    // (j - 2 + LAV) % NSTV == (j - 3) % NSTV
        FA_RING_CHECK(i, j3, v_read, 0);
        if (my_lo <= i - 1 && i - 1 <= my_hi) pv_plain(v_read);
        if (my_lo <= i && i <= my_hi) softmax_plain(i);
        if (my_lo <= i + 1 && i + 1 <= my_hi) qk_plain(j3, i + 1);
        FA_RING_CHECK(i, j3, v_read, 3);
        finish_iteration(more_k, more_v, tv > t1);
    };
    auto steady_iteration = [&](auto J3, int i, int jv) __attribute__((always_inline)) {
        constexpr int j3 = decltype(J3)::value;
        constexpr int jm1 = (j3 + NST - 1) % NST, jm2 = (j3 + 2 * NST - 2) % NST, jm3 = (j3 + 3 * NST - 3) % NST;
        const int tk = i + 1 + LA, tv = i - 1 + LAV;
        const bool more_k = tk <= t1, more_v = tv >= t0 && tv <= t1;
        const int v_read = NSTV == NST ? jm2 : jv, v_fill = NSTV == NST ? jm3 : (jv == 0 ? NSTV - 1 : jv - 1);
        if (NSTV < NST && more_v) issue_v(tv, v_fill);
#ifdef FA_CHECK_RING_BREAK
        // the checker's negative control: the K tile goes into the stage that is being read in this iteration
        if (more_k) issue_k(tk, j3);
#else
        if (more_k) issue_k(tk, jm1);
#endif
        if (NSTV == NST && more_v) issue_v(tv, v_fill);
        FA_RING_CHECK(i, j3, v_read, 1);
        steady(IntC<j3>{}, IntC<jm2>{}, v_read, i);
        FA_RING_CHECK(i, j3, v_read, 5);
        finish_iteration(more_k, more_v, false);
    };
    // jv: the V stage the iteration reads, (j - 2) mod NSTV, kept as a run-time counter (used when NSTV != NST)
    int i = t0 - 1, j3 = 0, jv = (2 * NSTV - 2) % NSTV;
    auto advance = [&]() __attribute__((always_inline)) {
        j3 = j3 == NST - 1 ? 0 : j3 + 1;
        jv = jv == NSTV - 1 ? 0 : jv + 1;
    };
    // An iteration in which this wave has all three pieces runs the interleaved body, whatever stage the ring is
    // at: single iterations in front of and behind the loop over whole turns of the ring bring the stage to 0 and
    // take what is left over (as plain pieces these iterations cost short problems 1-3 %).  Straight-line copies
    // on purpose: one loop that picks the body by the stage makes the register allocator spill 330-520 bytes.
    auto whole = [&](int it) __attribute__((always_inline)) { return it >= my_lo + 1 && it + 1 <= my_hi; };
    for (; i < t1; ++i) {                 // fill: until this wave has all three pieces of an iteration
        if (whole(i)) break;
        generic_iteration(i, j3, jv);
        advance();
    }
    if (j3 == 1 && whole(i)) { steady_iteration(IntC<1>{}, i, jv); advance(); ++i; }
    if (NST >= 3 && j3 == 2 && whole(i)) { steady_iteration(IntC<2 % NST>{}, i, jv); advance(); ++i; }
    for (; j3 == 0 && whole(i) && whole(i + NST - 1); i += NST) {
        steady_iteration(IntC<0>{}, i, jv);
        advance();
        steady_iteration(IntC<1>{}, i + 1, jv);
        advance();
        if (NST >= 3) { steady_iteration(IntC<2 % NST>{}, i + 2, jv); advance(); }
    }
    if (j3 == 0 && whole(i)) { steady_iteration(IntC<0>{}, i, jv); advance(); ++i; }
    if (NST >= 3 && j3 == 1 && whole(i)) { steady_iteration(IntC<1>{}, i, jv); advance(); ++i; }
    for (; i < t1; ++i) {                 // drain, up to the last two iterations
        generic_iteration(i, j3, jv);
        advance();
    }
    // Queue schedule: the counter round trip for the NEXT item (2.3 us) runs behind the last two iterations.
    // (Between two loops on purpose: as a branch inside generic_iteration the same statement costs the whole
    // kernel fifty registers.)
    if (a.queue != nullptr && tid == 0) ticket_ahead = atomicAdd(&a.queue[xcd], 1u);
    for (; i <= t1 + 1; ++i) {            // the last two iterations (three stages each: they request nothing any more)
        generic_iteration(i, j3, jv);
        advance();
    }

    }   // any_tile
    // rows 0..31 of a causal head are written by faithful_first_rows below instead (with key splits: in the
    // split that holds their keys, the first one; the others see none of their keys and write empty partials)
    // (GENERAL: query i sits at key position i + pos_off, so the rows concerned are those with i + pos_off < 32
    // (with more queries than keys, pos_off < 0, the path is not taken);
    // fa_fwd_params.exact_first_rows switches the path off)
    const bool first_rows_on = MASKED && a.R == 0 && pos_off >= 0 && pos_off < kFaithfulRows && split == 0 && pack == 1 && !a.exact_first_rows;
    const bool faithful = first_rows_on && q0 == 0;         // this item's own rows 0..31 are not stored by the epilogue
    const int f_rows = !faithful ? 0 : !GENERAL ? kFaithfulRows : (kFaithfulRows - pos_off < S ? kFaithfulRows - pos_off : S);
    // Which of those rows THIS item recomputes.  General layouts: the item with the head's first block, all of
    // them.  Contiguous layout: the 32 rows are dealt in 2, 4 or 8 parts to the head's first query blocks, one
    // part each -- under a static schedule the workgroups that run the path are the critical path of a short
    // problem (c2: 64 of 256 workgroups carried 7.7 us each), and every pair of items of the snake then gets one:
    // as many parts as half the head's blocks (at most eight), since the snake pairs block n - 1 with 0, n - 2 with
    // 1, ...  (Eight parts instead of four at sixteen blocks: c2 592.7 against 584.4 TFLOP/s, B4 H32 S2048 D64 654.7
    // against 641.7; two parts instead of four at four blocks, where four gave every pair two of them: causal B16 H16
    // S512 D128 380.1 against 359.3, D64 276.8 against 266.3.)  One workgroup per item and the work queue, which
    // balances by itself, keep four parts.
    int fr0 = 0, fr1 = 0;
    // (general layouts deal the rows the same way when the problem is the plain one at another length: queries
    // that start at key position 0, no key splits; otherwise the item with the head's first block keeps them all)
    // (causal B8 H32 S1000 D64 445 against 382 TFLOP/s, B16 H16 S500 D128 341 against 296, B4 H16 S2047 D64 573 against
    // 521.  The general 4-wave kernels keep two LDS stages per tensor: with three for K their 128-wide instantiations
    // spill 24-40 bytes and measure 3-5 % slower.)
    const bool dealt = !GENERAL || (n_splits == 1 && pos_off == 0 && a.n_qblocks >= 2);
    if (!dealt) fr1 = f_rows;
    else if (first_rows_on) {
        // (a resident grid without a queue walks the list as a snake: a workgroup's items come in pairs of block k
        // and block n - 1 - k, and parts on the lower half of the blocks give every pair exactly one)
        const bool snake = a.queue == nullptr && (long long)gridDim.x < a.n_items;
        const int parts = snake ? (a.n_qblocks >= 16 ? 8 : a.n_qblocks >= 8 ? 4 : a.n_qblocks >= 4 ? 2 : 1)
                                : (a.n_qblocks >= 4 ? 4 : a.n_qblocks >= 2 ? 2 : 1);
        if (qblock < parts) { fr0 = qblock * (kFaithfulRows / parts); fr1 = fr0 + kFaithfulRows / parts; }
    }
    // ---- the next work item, and the first requests for it
    const int next_item = take_item(pass + 1, ticket_ahead);
    // (the first-rows path below works in the LDS behind the K stages that are filled here)
    if (!GENERAL && next_item >= 0) {
        int nbh, nqb, nt0, nt1;
        fa_item_decode(next_item, a.BH, a.n_qblocks, a.descending, &nbh, &nqb);
        const uint16_t *nQ, *nK, *nV;
        if (STRIDED) {
            int nhi, nhk;
            const int nbi = fa_strided_heads(nbh, a.H, a.Hk, &nhi, &nhk);
            nQ = a.Q + (size_t)nbi * a.q_bs + (size_t)nhi * a.q_hs;
            nK = a.K + (size_t)nbi * a.k_bs + (size_t)nhk * a.k_hs;
            nV = a.V + (size_t)nbi * a.v_bs + (size_t)nhk * a.v_hs;
        } else {
            const size_t noff = (size_t)nbh * S * D;
            nQ = a.Q + noff; nK = a.K + noff; nV = a.V + noff;
        }
        const int nq0 = nqb * BR;
        fa_tile_range(S, kBlockKeys, a.L, a.R, nq0, S - nq0 < BR ? S - nq0 : BR, &nt0, &nt1);
        // (every LDS stage is free: the last iteration ended with a barrier)
        issue_k_from(nK, nt0, 0);
        if (LA > 1 && nt0 + 1 <= nt1) issue_k_from(nK, nt0 + 1, 1);
        // (S is a multiple of 128: a wave has all its rows or none; one without rows never uses its fragments and
        // reads those of the block's first wave, so that no select has to wait for the data)
        const int nrow = nq0 + (nq0 + wave * WR < S ? wave * WR : 0) + l32;
#pragma unroll
        for (int s = 0; s < KS; ++s)
            qf[s] = *reinterpret_cast<const u32x4 *>(nQ + (size_t)nrow * q_rs + 16 * s + 8 * half);
        next_requested = true;
    }
    // With key splits the item writes fp32 partial results, (O normalised over its own keys, logsumexp of its
    // own keys), which fa_combine_splits merges.
    float *o_part = nullptr, *lse_part = nullptr;
    if (GENERAL && n_splits > 1) {
        const size_t part = (size_t)split * a.BH + bh;       // (row_head rows further for the heads of a packed group)
        o_part = a.o_part + part * S * D;
        lse_part = a.lse_part + part * S;
    }
    // ---- epilogue: O / l, logsumexp (the reference has none; flash_forward.h:318-327 only divides).  Not for a
    // row past the end, nor for rows that faithful_first_rows writes below.
    const bool own_store = wave_live && row_ok && !(!GENERAL && faithful && wave == 0) && !(GENERAL && my_q < f_rows);
    if (own_store) {
        {
            // the row's index in its head's [S, ...] output, counted from head `bh` (packed groups: row_head
            // heads further on; their logsumexp and partial rows follow at S per head, their O rows at o_hs)
            const int q = GENERAL ? row_head * S + row_pos : my_q;
            const float l_half = l_a + l_b;
            const float l_tot = l_half + swap_halves(l_half);
            const bool empty = GENERAL && !(l_tot > 0.0f);         // this row saw no key (here)
            const float inv = empty ? 0.0f : (DROPOUT ? a.drop_scale : 1.0f) / l_tot;
            const float lse_row = empty ? -INFINITY
                                        : m_run * a.scale + __builtin_logf(l_tot);
            if (GENERAL && o_part != nullptr) {
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const f32x4 w = {o[db][4 * g] * inv, o[db][4 * g + 1] * inv, o[db][4 * g + 2] * inv,
                                         o[db][4 * g + 3] * inv};
                        *reinterpret_cast<f32x4 *>(o_part + (size_t)q * D + 32 * db + 8 * g + 4 * half) = w;
                    }
                if (half == 0) lse_part[q] = lse_row;
            } else if (!GENERAL) {
                // Through LDS, so that every store instruction writes whole rows: a lane holds 8-byte pieces of ONE
                // row, and stored from the registers an instruction touches 32 rows with 16 bytes each (the
                // address path takes as long for it as for 32 full cache lines); row-major, four (eight) rows of
                // 256 (128) bytes per instruction.  The wave's 32 x D block sits in LDS that nothing else uses at
                // this point (behind the K stages that the requests for the next item fill), 16-byte chunks
                // XOR-swizzled by the row; written and read by this wave only, whose LDS operations complete in order.
                typedef __attribute__((address_space(3))) u32x2 lds_u32x2;
                typedef __attribute__((address_space(3))) u32x4 lds_u32x4;
                // (the lane index is taken from the hardware here and tied to this place: derived from threadIdx.x,
                // these addresses are formed at the top of the kernel and kept in registers through the tile loop)
                int lane_e = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
                asm volatile("" : "+v"(lane_e));
                const int l32_e = lane_e & 31, half_e = lane_e >> 5;
                const uint32_t obase = lds0 + LA * TILEB + wave * (32 * ROWB);
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        u32x2 w;
                        w[0] = N::pack2(o[db][4 * g] * inv, o[db][4 * g + 1] * inv);
                        w[1] = N::pack2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
                        const int chunk = 4 * db + g;           // 16-byte chunk of the row: elements 8 * chunk .. + 7
                        *(lds_u32x2 *)(uintptr_t)(obase + l32_e * ROWB + ((chunk ^ (l32_e & (CPR - 1))) << 4) + 8 * half_e) = w;
                    }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                constexpr int RPI = 64 / CPR;                   // rows per store instruction
#pragma unroll
                for (int i = 0; i < 32 / RPI; ++i) {
                    const int row = RPI * i + lane_e / CPR, chunk = lane_e % CPR;
                    const u32x4 w = *(const lds_u32x4 *)(uintptr_t)(obase + row * ROWB + ((chunk ^ (row & (CPR - 1))) << 4));
                    *reinterpret_cast<u32x4 *>(Oh + (size_t)(qw + row) * o_rs + 8 * chunk) = w;
                }
            } else {
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    u32x2 w;
                    w[0] = N::pack2(o[db][4 * g] * inv, o[db][4 * g + 1] * inv);
                    w[1] = N::pack2(o[db][4 * g + 2] * inv, o[db][4 * g + 3] * inv);
                    *reinterpret_cast<u32x2 *>(Oh + (GENERAL ? (size_t)row_head * a.o_hs + (size_t)row_pos * o_rs : (size_t)q * o_rs) +
                                               32 * db + 8 * g + 4 * half) = w;
                }
            }
            if (!(GENERAL && o_part != nullptr) && a.lse != nullptr && half == 0) a.lse[(size_t)bh * S + q] = lse_row;
        }
    }
    if (!GENERAL && fr1 > fr0) __syncthreads();       // (the epilogue's LDS blocks have been read by their waves)
    if (fr1 > fr0)    // the LDS behind the first LA K stages is free
        faithful_first_rows<BF16, D>(Qh, Kh, Vh, Oh, o_part, o_part != nullptr ? lse_part : a.lse != nullptr ? a.lse + (size_t)bh * S : nullptr,
                                     fr0, fr1, pos_off, a.L, a.scale, slope, q_rs, k_rs, v_rs, o_rs, DROPOUT ? a.drop_threshold : 0u, a.drop_scale,
                                     a.seed_lo, a.seed_hi, (uint32_t)bh, lds0 + LA * TILEB);
    item = next_item;
    }   // next work item
    // the last workgroup to leave rewinds the queue for the next launch that uses it
    if (a.queue != nullptr && tid == 0) {
        __threadfence();
        if (atomicAdd(&a.queue[8], 1u) == (unsigned)G - 1u) {
#pragma unroll
            for (int x = 0; x < 9; ++x) a.queue[x] = 0u;
        }
    }
}

// Merges the partial results of a launch with key splits: for every query row,
//   LSE = log sum_s exp(LSE_s),  O = sum_s exp(LSE_s - LSE) * O_s
// (a split that saw no key of the row has LSE_s = -inf and weight 0).  One thread per four output elements.
template <bool BF16, int D>
__global__ void __launch_bounds__(256) fa_combine_splits(const FaKernelArgs a)
{
    constexpr int TPR = D / 4;                    // threads per row
    const long long row = (long long)blockIdx.x * (256 / TPR) + threadIdx.x / TPR;
    const int c4 = (threadIdx.x % TPR) * 4;
    const long long n_rows = (long long)a.BH * a.S;
    if (row >= n_rows) return;
    const int bh = (int)(row / a.S), q = (int)(row % a.S);
    float mx = -INFINITY;
    for (int s = 0; s < a.n_splits; ++s) mx = fmaxf(mx, a.lse_part[(size_t)s * n_rows + row]);
    float wsum = 0.0f;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (mx != -INFINITY) {
        for (int s = 0; s < a.n_splits; ++s) {
            const float w = __expf(a.lse_part[(size_t)s * n_rows + row] - mx);
            if (w > 0.0f) {
                const f32x4 o = *reinterpret_cast<const f32x4 *>(a.o_part + ((size_t)s * n_rows + row) * D + c4);
                acc += o * w;
                wsum += w;
            }
        }
        acc *= 1.0f / wsum;
    }
    const int bi = bh / a.H, hi = bh - bi * a.H;
    uint16_t *dst = a.O + (size_t)bi * a.o_bs + (size_t)hi * a.o_hs + (size_t)q * a.o_rs + c4;
    u32x2 w2;
    w2[0] = Num<BF16>::pack2(acc[0], acc[1]);
    w2[1] = Num<BF16>::pack2(acc[2], acc[3]);
    *reinterpret_cast<u32x2 *>(dst) = w2;
    if (a.lse != nullptr && c4 == 0) a.lse[row] = mx == -INFINITY ? -INFINITY : mx + __logf(wsum);
}

template <bool BF16, int D, bool MASKED, bool ALIBI, bool GENERAL, bool DROPOUT, int NW, int NST, bool STRIDED = false, int NSTV = NST>
hipError_t launch(const FaKernelArgs &a, unsigned grid, hipStream_t stream, bool configure_only)
{
    constexpr int TILEB = kBlockKeys * D * 2;
    const size_t smem = (NST + NSTV) * TILEB;      // the stages (the queue schedule's word borrows the last bytes between items)
    auto kern = fa_fwd_pipelined<BF16, D, MASKED, ALIBI, GENERAL, DROPOUT, NW, NST, STRIDED, NSTV>;
    // the LDS opt-in is per (instantiation, device) and is made once, not on every launch
    static std::atomic<unsigned long long> configured{0ull};
    const unsigned long long dev_bit = 1ull << fa_launch_device();
    if (!(configured.load(std::memory_order_relaxed) & dev_bit)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
        if (e != hipSuccess) return e;
        configured.fetch_or(dev_bit, std::memory_order_relaxed);
    }
    if (configure_only) return hipSuccess;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), smem, stream, a);
    return hipGetLastError();
}


// shape 0: 8 waves x 32 rows = 256 query rows per workgroup, three LDS stages, one workgroup per CU.
// shape 1: 4 waves x 32 rows = 128 query rows per workgroup, two LDS stages, two workgroups per CU.
// (The 8-wave general instantiations get two LDS stages instead of three: a third buys nothing measurable --
// c3's shape stored [B,S,H,D] runs at 925 TFLOP/s with two and 929 with three, c2's at 553 against 514 -- and
// two leave LDS for a second workgroup of the small shapes.)
template <bool GENERAL, bool DROPOUT, bool STRIDED = false>
hipError_t launch_forward(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid, hipStream_t stream,
                          bool configure_only = false)
{
    const int alibi = a.alibi != nullptr;
#define FA_CASE(BF, DD, MK, AL) \
    if (bf16 == BF && D == DD && masked == MK && alibi == AL) { \
        if (shape == 0) return launch<BF != 0, DD, MK != 0, AL != 0, GENERAL, DROPOUT, 8, (GENERAL ? 2 : 3), STRIDED>(a, grid, stream, configure_only); \
        return launch<BF != 0, DD, MK != 0, AL != 0, GENERAL, DROPOUT, 4, (GENERAL ? 2 : FA_S1K), STRIDED, (GENERAL ? 2 : FA_S1V)>(a, grid, stream, configure_only); \
    }
#define FA_CASES(BF, DD) FA_CASE(BF, DD, 0, 0) FA_CASE(BF, DD, 1, 0) FA_CASE(BF, DD, 0, 1) FA_CASE(BF, DD, 1, 1)
    FA_CASES(0, 64) FA_CASES(0, 128) FA_CASES(1, 64) FA_CASES(1, 128)
#undef FA_CASES
#undef FA_CASE
    return hipErrorInvalidValue;
}

// The LDS opt-in of every instantiation of one flavour, for the current device, without launching anything: what
// fa_init() runs so that no later launch has to (hipFuncSetAttribute is not a stream operation and must not
// fall into a stream capture).
template <bool GENERAL, bool DROPOUT, bool STRIDED = false>
hipError_t configure_forward()
{
    FaKernelArgs a = {};
    static const float slope_stand_in = 0.0f;      // (only tested against null)
    for (int bf16 = 0; bf16 < 2; ++bf16)
        for (int D = 64; D <= 128; D += 64)
            for (int masked = 0; masked < 2; ++masked)
                for (int alibi = 0; alibi < 2; ++alibi)
                    for (int shape = 0; shape < 2; ++shape) {
                        a.alibi = alibi ? &slope_stand_in : nullptr;
                        const hipError_t e = launch_forward<GENERAL, DROPOUT, STRIDED>(a, bf16, D, masked, shape, 0u, nullptr, true);
                        if (e != hipSuccess) return e;
                    }
    return hipSuccess;
}

}  // namespace

#endif
