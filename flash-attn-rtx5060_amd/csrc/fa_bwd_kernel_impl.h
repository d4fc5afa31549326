// FlashAttention backward for gfx950 (MI355X): dQ, dK, dV from Q, K, V, O, dO and the logsumexp the forward
// pass writes.  The reference has no backward pass (its L output is accepted and never written, reference
// src/flash_forward.h:602,628-644); this is the consumer of the logsumexp this library emits.
//
//   P  = exp(scale * Q K^T - LSE)            (recomputed; masked pairs are 0)
//   dV = P^T dO
//   dP = dO V^T,   delta_i = sum_t dO_it O_it
//   dS = P o (dP - delta)
//   dQ = scale * dS K,   dK = scale * dS^T Q
//
// Two kernels: fa_bwd_dq (a workgroup owns 256 queries and walks the key tiles; it also writes delta and the
// rescaled logsumexp for the second kernel) and fa_bwd_dkdv (a workgroup owns 256 keys of one K/V head and walks
// the query tiles of the query heads that share it); no atomics, every output element has one writer, results
// are the same bits from run to run.
// Template flags: LAYOUT 0 = contiguous [B,H,S,D] with S a multiple of 128 and as many keys; 1 (strided) = the
// same lengths with row, head and batch strides from the arguments and grouped K/V heads; 2 (general) = that
// plus any lengths (query i at key position i + Sk - S, ragged last tiles).  Each keeps its instruction stream
// free of what it does not need.  ALIBI subtracts slope[h] * |position - key| from the scaled score.  DROPOUT
// replays the forward pass's keep decisions from (seed, head, query position, key).  (Either one is instantiated
// for all three layouts, both together for the general one only.)
// Layouts 0 and 1 also have a five-product form (fa_bwd_prepare, fa_bwd_dkdv<WRITE_DS>, fa_bwd_dq_from_ds below).
// Both walkers use the building blocks of the forward kernel: 32x32x16 MFMA with the thing a wave owns on the
// lane (query in fa_bwd_dq, key in fa_bwd_dkdv), so that the owner's operands are B operands loaded once into
// registers, the walked tiles are A operands streamed through LDS by direct global->LDS loads, and an
// accumulator tile is already laid out as the B operand of the next product.
// A walked tile that is needed both row-wise (ds_read_b128) and transposed (ds_read_b64_tr_b16) sits in LDS
// once, under a swizzle that is bank-conflict-free for both.
#ifndef FA_BWD_KERNEL_IMPL_H
#define FA_BWD_KERNEL_IMPL_H
#include "fa_fwd_kernel_impl.h"
#include "fa_bwd_args.h"
#include "fa_bwd_layout.h"

#ifndef FA_DS_LOOP
#define FA_DS_LOOP 1
#endif
#ifndef FA_PARK_DROP
#define FA_PARK_DROP 3
#endif
namespace {

constexpr int kBwdWaves = 8;            // 8 waves x 32 owned rows = 256 rows per workgroup, two waves per SIMD
constexpr int kBwdStages = 3;           // LDS ring: with three stages one barrier per tile is enough
constexpr float kLog2e = 1.44269504088896340736f;
constexpr int kDsBlockBytes = 2048;     // one 32-query x 32-key block of dS in the storage type

// Takes the word by value on purpose: __builtin_bit_cast applied directly to an element of a vector
// (`__builtin_bit_cast(float, v[e])`) reads element 0 whatever e is with this compiler.
__device__ __forceinline__ float as_f32(uint32_t w) { return __builtin_bit_cast(float, w); }

// per-lane LDS addresses of the two read patterns in the stage being read; everything else about a fragment
// (which of the stage's tiles, which 32-row block, which 16-row slice) is an immediate offset of the read
template <int D> struct TileReader {
    static constexpr int CPR = D / 8, ROWB = D * 2, KS = D / 16, DB = D / 32;
    uint32_t row_addr[KS];      // ds_read_b128: A operand rows = tile rows, k = 16 head-dim values of slice s
    uint32_t tr_addr[DB][2];    // ds_read_b64_tr_b16: A operand rows = head dim (block db), k = 16 tile rows (two reads of 8)
    __device__ __forceinline__ void init(int lane, uint32_t stage_base)
    {
#pragma unroll
        for (int s = 0; s < KS; ++s) row_addr[s] = stage_base + (uint32_t)fa_bwd_row_read(D, lane, s);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int hi = 0; hi < 2; ++hi) tr_addr[db][hi] = stage_base + (uint32_t)fa_bwd_tr_read(D, lane, db, hi);
    }
    // move to another stage of the ring (delta in bytes, wave-uniform)
    __device__ __forceinline__ void advance(int delta)
    {
#pragma unroll
        for (int s = 0; s < KS; ++s) row_addr[s] += delta;
#pragma unroll
        for (int db = 0; db < DB; ++db) { tr_addr[db][0] += delta; tr_addr[db][1] += delta; }
    }
    // row-wise fragment: head-dim slice s, 32-row block b of the tile at byte `tile` of the stage
    __device__ __forceinline__ u32x4 rows(int tile, int s, int b) const { return lds_read_b128(row_addr[s] + (uint32_t)(tile + b * 32 * ROWB)); }
    // transposed fragment: 16-row slice t2, head-dim block db of the tile at byte `tile` of the stage
    __device__ __forceinline__ u32x4 transposed(int tile, int t2, int db) const
    {
        const u32x2 lo = lds_read_tr(tr_addr[db][0] + (uint32_t)(tile + (16 * t2) * ROWB));
        const u32x2 hi = lds_read_tr(tr_addr[db][1] + (uint32_t)(tile + (16 * t2) * ROWB));
        return u32x4{lo[0], lo[1], hi[0], hi[1]};
    }
};

// one 64-row tile global -> LDS: wave w issues instructions w, w+8, ...
template <int D> struct TileLoader {
    static constexpr int CPR = D / 8, ROWB = D * 2, TILEB = 64 * ROWB, IPW = TILEB / 1024 / kBwdWaves;
    uint32_t g[IPW];
    int wave, lane;
    // row_bytes: distance between consecutive rows of the source in bytes
    __device__ __forceinline__ void init(int wave_, int lane_, int row_bytes)
    {
        wave = wave_; lane = lane_;
#pragma unroll
        for (int i = 0; i < IPW; ++i) {
            g[i] = (uint32_t)fa_bwd_load_source(D, (i * kBwdWaves + wave) * 64 + lane, row_bytes);
        }
    }
    __device__ __forceinline__ void load(const uint16_t *tile_src, uint32_t lds_tile) const
    {
#pragma unroll
        for (int i = 0; i < IPW; ++i)
            dma_16(reinterpret_cast<const char *>(tile_src), g[i], lds_tile + (i * kBwdWaves + wave) * 1024);
    }
    // a tile whose last rows lie past the end of the tensor: they are filled with copies of row `valid - 1`
    __device__ __forceinline__ void load_ragged(const uint16_t *tile_src, uint32_t lds_tile, int valid, int row_bytes) const
    {
        // (the empty asm keeps the address arithmetic of this rare path inside its branch: hoisted out of the
        // tile loop it would occupy registers for the whole kernel)
        int ln = lane;
        asm volatile("" : "+v"(ln));
#pragma unroll
        for (int i = 0; i < IPW; ++i) {
            const int P = (i * kBwdWaves + wave) * 64 + ln, row = P / CPR, pos = P % CPR;
            const int src_row = row < valid ? row : valid - 1;
            dma_16(reinterpret_cast<const char *>(tile_src), (uint32_t)(src_row * row_bytes + ((pos ^ fa_u_swz(CPR, row)) << 4)),
                   lds_tile + (i * kBwdWaves + wave) * 1024);
        }
    }
};

// 256 bytes (64 floats) global -> LDS in one wave instruction: lane l copies the float at src[index] to LDS
// byte lds + 4*l
__device__ __forceinline__ void dma_4(const float *src, int index, uint32_t lds)
{
    const uint64_t b = (uint64_t)src;
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint64_t ub = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
    const uint32_t voff = (uint32_t)index * 4u;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds)), "v"(voff), "s"(ub) : "memory", "m0");
}

// s_waitcnt vmcnt(n) for a wave-uniform run-time n (the instruction takes an immediate)
__device__ __forceinline__ void wait_vm_upto(int n)
{
    switch (n) {
#define FA_WAIT_CASE(k) case k: wait_vm<k>(); break;
    FA_WAIT_CASE(0) FA_WAIT_CASE(1) FA_WAIT_CASE(2) FA_WAIT_CASE(3) FA_WAIT_CASE(4) FA_WAIT_CASE(5) FA_WAIT_CASE(6) FA_WAIT_CASE(7)
    FA_WAIT_CASE(8) FA_WAIT_CASE(9) FA_WAIT_CASE(10) FA_WAIT_CASE(11) FA_WAIT_CASE(12) FA_WAIT_CASE(13) FA_WAIT_CASE(14) FA_WAIT_CASE(15)
    FA_WAIT_CASE(16)
#undef FA_WAIT_CASE
    default: wait_vm<0>(); break;
    }
}

// dma_16 with the streaming hint: data that is read exactly once should not displace what others re-read from L2
__device__ __forceinline__ void dma_16_stream(const char *base, uint32_t voff, uint32_t lds)
{
    const uint64_t b = (uint64_t)base;
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint64_t ub = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds)), "v"(voff), "s"(ub) : "memory", "m0");
}

__device__ __forceinline__ f32x16 zero16()
{
    f32x16 z;
#pragma unroll
    for (int r = 0; r < 16; ++r) z[r] = 0.0f;
    return z;
}

// The kernel's arguments, read again from the kernel-argument segment: what is taken from the by-value argument
// is loaded once in front of the item loop and then kept in scalar registers through every tile loop; a use behind
// this call loads it where it is needed (scalar loads from a segment that stays in the scalar cache).
__device__ __forceinline__ const FaBwdArgs &args_reloaded()
{
    typedef const __attribute__((address_space(4))) FaBwdArgs *KernargPtr;
    KernargPtr ka = (KernargPtr)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(ka));
    return *(const FaBwdArgs *)ka;
}

__device__ __forceinline__ const uint16_t *head_ptr(const uint16_t *p, const FaBwdTensor &t, int b, int h)
{
    return p + (long long)b * t.bs + (long long)h * t.hs;
}
__device__ __forceinline__ uint16_t *head_ptr(uint16_t *p, const FaBwdTensor &t, int b, int h)
{
    return p + (long long)b * t.bs + (long long)h * t.hs;
}

// ---------------------------------------------------------------------------------------------------------
// dQ: a workgroup owns 256 queries (lane = query), walks the key tiles of its visible range.
// LDS stage: K (read row-wise for S^T = K Q^T and transposed for dQ^T += K^T dS^T), V (row-wise, dP^T = V dO^T).
// ---------------------------------------------------------------------------------------------------------
template <bool BF16, int D, bool MASKED, int LAYOUT, bool ALIBI, bool DROPOUT>
__global__ void __launch_bounds__(kBwdWaves * 64, 2) fa_bwd_dq(const FaBwdArgs a)
{
    constexpr bool STRIDES = LAYOUT >= 1, GENERAL = LAYOUT == 2, ONE_ITEM = STRIDES && D == 128;
    static_assert(LAYOUT >= 0 && LAYOUT <= 2, "0 the reference's layout, 1 strided, 2 general");
    static_assert(!GENERAL || MASKED, "the general instantiations always carry the mask code (ragged tiles need it)");

    typedef Num<BF16> N;
    typedef TileReader<D> Reader;
    typedef TileLoader<D> Loader;
    constexpr int KS = Reader::KS, DB = Reader::DB, TILEB = Loader::TILEB, STAGEB = 2 * TILEB, IPW = Loader::IPW;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int S = a.S, Sk = GENERAL ? a.Sk : a.S, off = GENERAL ? a.Sk - a.S : 0;
    const int n_qblocks = (S + 255) / 256;
    // one head per XCD at a time, long blocks first: the workgroups that share a head's K and V share an L2
    // Work items: one workgroup per item, or (grid smaller than the list) a resident grid that walks the
    // longest-first list as a snake, pass 0 forwards, pass 1 backwards, ..., which pairs long items with short ones.
    const long long n_items = (long long)a.B * a.H * n_qblocks;
    for (int pass = 0; !ONE_ITEM || pass < 1; ++pass) {       // (128-wide strided and general instantiations: exactly one item, no loop)
    const long long item = (long long)pass * gridDim.x + ((pass & 1) ? gridDim.x - 1 - blockIdx.x : blockIdx.x);
    if (item >= n_items) break;
    if (pass > 0) __syncthreads();          // (the LDS stages: other waves may still be reading the last tile)
    // (the lane index is taken from the hardware once per work item and tied to this place: what is derived from
    // it would otherwise be computed in front of the item loop and kept in registers through every tile loop)
    int lane = ONE_ITEM ? (int)threadIdx.x & 63 : (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    if (!ONE_ITEM) asm volatile("" : "+v"(lane));
    const int half = lane >> 5, l32 = lane & 31;
    int bh, qblock;
    fa_item_decode(item, a.B * a.H, n_qblocks, MASKED ? 1 : 0, &bh, &qblock);
    const int b = bh / a.H, h = bh - b * a.H, hk = STRIDES ? h / (a.H / a.Hk) : h;
    const int q_rs = STRIDES ? a.q.rs : D, k_rs = STRIDES ? a.k.rs : D, v_rs = STRIDES ? a.v.rs : D;
    const int o_rs = STRIDES ? a.o.rs : D, g_rs = STRIDES ? a.dO_.rs : D, dq_rs = STRIDES ? a.dq.rs : D;
    const uint16_t *Qh, *Kh, *Vh, *Oh, *dOh;
    uint16_t *dQh;
    if (STRIDES) {
        Qh = head_ptr(a.Q, a.q, b, h); Kh = head_ptr(a.K, a.k, b, hk); Vh = head_ptr(a.V, a.v, b, hk);
        Oh = head_ptr(a.O, a.o, b, h); dOh = head_ptr(a.dO, a.dO_, b, h); dQh = head_ptr(a.dQ, a.dq, b, h);
    } else {
        const size_t head_off = (size_t)bh * S * D;
        Qh = a.Q + head_off; Kh = a.K + head_off; Vh = a.V + head_off; Oh = a.O + head_off; dOh = a.dO + head_off;
        dQh = a.dQ + head_off;
    }
    const int q0 = qblock * 256, qw = q0 + wave * 32;
    const bool active = qw < S;                    // the last block may own fewer than 256 rows
    const int my_q = active ? (GENERAL && qw + l32 >= S ? S - 1 : qw + l32) : (GENERAL ? 0 : l32);   // row to load
    const bool row_ok = active && qw + l32 < S;
    const int my_pos = qw + l32 + off;             // key position of this lane's query (masks, ALiBi)

    u32x4 qf[KS], gf[KS];           // Q^T and dO^T as B operands: lane = (query, head-dim slice 8*half..+7 of each 16)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        qf[s] = *reinterpret_cast<const u32x4 *>(Qh + (size_t)my_q * q_rs + 16 * s + 8 * half);
        gf[s] = *reinterpret_cast<const u32x4 *>(dOh + (size_t)my_q * g_rs + 16 * s + 8 * half);
    }
    // logsumexp in exp2 units; a row that saw no key has -inf there and takes +inf here, which makes every P 0
    const float lse_raw = a.lse[(size_t)bh * S + my_q];
    float lse_l2 = (GENERAL && lse_raw == -INFINITY) ? INFINITY : lse_raw * kLog2e;
    // delta_i = sum_t dO_it O_it: this lane holds half of row i of dO already; the other half is on lane ^ 32.
    // Both are written out for fa_bwd_dkdv, which runs after this kernel.
    float delta = 0.0f;
    {
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            const u32x4 o = *reinterpret_cast<const u32x4 *>(Oh + (size_t)my_q * o_rs + 16 * s + 8 * half);
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const uint32_t ow = o[w], gw = gf[s][w];
                delta += storage_to_f32<BF16>((uint16_t)(ow & 0xffffu)) * storage_to_f32<BF16>((uint16_t)(gw & 0xffffu));
                delta += storage_to_f32<BF16>((uint16_t)(ow >> 16)) * storage_to_f32<BF16>((uint16_t)(gw >> 16));
            }
        }
        delta += swap_halves(delta);
        if (row_ok && half == 0) {
            a.delta[(size_t)bh * S + my_q] = delta;
            a.lse2[(size_t)bh * S + my_q] = lse_l2;
        }
    }
    const float c = a.scale * kLog2e;
    float slope_l2 = 0.0f;
    if (ALIBI) slope_l2 = a.alibi[h] * kLog2e;

    int t0, t1, my_lo = 1, my_hi = 0;
    fa_tile_range(Sk, 64, a.L, a.R, q0 + off, S - q0 < 256 ? S - q0 : 256, &t0, &t1);
    if (active) fa_tile_range(Sk, 64, a.L, a.R, qw + off, GENERAL && S - qw < 32 ? S - qw : 32, &my_lo, &my_hi);

    Reader rd; rd.init(lane, lds0);
    Loader ldk, ldv;
    ldk.init(wave, lane, k_rs * 2);
    if (STRIDES) ldv.init(wave, lane, v_rs * 2);
    auto issue = [&](int tile, int stage) __attribute__((always_inline)) {
        const uint32_t base = lds0 + stage * STAGEB;
        if (GENERAL && (tile + 1) * 64 > Sk) {
            ldk.load_ragged(Kh + (size_t)tile * 64 * k_rs, base, Sk - tile * 64, k_rs * 2);
            ldv.load_ragged(Vh + (size_t)tile * 64 * v_rs, base + TILEB, Sk - tile * 64, v_rs * 2);
        } else {
            ldk.load(Kh + (size_t)tile * 64 * k_rs, base);
            (STRIDES ? ldv : ldk).load(Vh + (size_t)tile * 64 * v_rs, base + TILEB);
        }
    };

    f32x16 dq[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) dq[db] = zero16();

    // 32 keys (block kb of the tile in the stage being read) against this wave's 32 queries
    auto half_tile = [&](bool edge, int t, int kb) __attribute__((always_inline)) {
        constexpr int k_tile = 0, v_tile = TILEB;
        f32x16 sx = zero16(), dp = zero16();
#pragma unroll
        for (int s = 0; s < KS; ++s) sx = N::mfma(rd.rows(k_tile, s, kb), qf[s], sx);      // S^T = K Q^T
#pragma unroll
        for (int s = 0; s < KS; ++s) dp = N::mfma(rd.rows(v_tile, s, kb), gf[s], dp);      // dP^T = V dO^T
        const int first = t * 64 + 32 * kb + 4 * half;                      // key of accumulator row 0 on this lane
        if (MASKED && edge) {            // wave-uniform; a masked score becomes -inf and its P exactly 0
            int hi = my_pos + a.R, lo = my_pos - a.L - first;                // visible: lo <= 8*(r/4) + r%4 <= hi
            if (GENERAL && hi > Sk - 1) hi = Sk - 1;
            hi -= first;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (8 * (r >> 2) + (r & 3) > hi || 8 * (r >> 2) + (r & 3) < lo) sx[r] = -INFINITY;
        }
        // dropout: the forward kept key j of this query iff byte r of this block is >= the threshold, and scaled
        // the kept probabilities; the same factor reaches dP, while the softmax Jacobian sees the undropped P
        DropWords dw;
        if (DROPOUT) dw = dropout_words(a.seed_lo, a.seed_hi, (uint32_t)bh, (uint32_t)my_pos, (uint32_t)(2 * (2 * t + kb) + half));
        uint32_t ds[8];                                  // dS^T in B-operand order
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float v[2];
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                const int r = 2 * i + e;
                float x = __builtin_fmaf(sx[r], c, -lse_l2);
                if (ALIBI) x = __builtin_fmaf(-slope_l2, __builtin_fabsf((float)(first + 8 * (r >> 2) + (r & 3) - my_pos)), x);
                const float p = __builtin_amdgcn_exp2f(x);
                float dpr = dp[r];
                if (DROPOUT) dpr = dropout_keep_byte(dw, r, a.drop_threshold) ? dpr * a.drop_scale : 0.0f;
                v[e] = p * (dpr - delta);
            }
            ds[i] = N::pack2(v[0], v[1]);
        }
#pragma unroll
        for (int n = 0; n < 2 * DB; ++n) {                // dQ^T += K^T dS^T
            const int h2 = n / DB, db = n % DB;
            const u32x4 bfrag = {ds[4 * h2], ds[4 * h2 + 1], ds[4 * h2 + 2], ds[4 * h2 + 3]};
            dq[db] = N::mfma(rd.transposed(k_tile, 2 * kb + h2, db), bfrag, dq[db]);
        }
    };

    if (t0 <= t1) {
        // Tiles are fetched two ahead: tile t+2 is issued at the end of iteration t, into the stage tile t-1 was
        // read from (free for everyone since this iteration's barrier).  A wait for "everything in flight" in the
        // middle of an iteration -- the compiler's own, around a register it spilled -- then only meets loads
        // that were issued a whole iteration earlier.
        issue(t0, 0);
        if (t0 + 1 <= t1) issue(t0 + 1, 1);
        wait_vm<0>();
        // the owner's operands have landed too: say so, or the compiler waits for them inside the loop, where
        // its wait would also cover the asynchronous tile loads
#pragma unroll
        for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]), "+v"(gf[s]));
        asm volatile("" : "+v"(lse_l2), "+v"(delta), "+v"(slope_l2));
        int stage = 0;
        for (int t = t0; t <= t1; ++t) {
            const int next = stage == kBwdStages - 1 ? 0 : stage + 1;
            if (t + 1 <= t1) wait_vm<2 * IPW>();                // tile t has landed, tile t+1 may still be in flight
            else wait_vm<0>();
            phase_barrier();                                    // tile t is in LDS for everyone; tile t-1's stage is free
            if (my_lo <= t && t <= my_hi) {
                const bool edge = MASKED && (fa_tile_class(64, a.L, a.R, qw + off, 32, t) == 1 || (GENERAL && (t + 1) * 64 > Sk));
                half_tile(edge, t, 0);
                half_tile(edge, t, 1);
            }
            if (t + 2 <= t1) issue(t + 2, next == kBwdStages - 1 ? 0 : next + 1);
            rd.advance(next == 0 ? -(kBwdStages - 1) * STAGEB : STAGEB);
            stage = next;
        }
    }
    if (row_ok) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 w;
                w[0] = N::pack2(dq[db][4 * g] * a.scale, dq[db][4 * g + 1] * a.scale);
                w[1] = N::pack2(dq[db][4 * g + 2] * a.scale, dq[db][4 * g + 3] * a.scale);
                *reinterpret_cast<u32x2 *>(dQh + (size_t)my_q * dq_rs + 32 * db + 8 * g + 4 * half) = w;
            }
    }
    }   // next work item
}

// ---------------------------------------------------------------------------------------------------------
// dK, dV: a workgroup owns 256 keys of one K/V head (lane = key), walks the query tiles that see them, for each
// of the query heads that share the K/V head.
// LDS stage: Q (row-wise for S = Q K^T, transposed for dK^T += Q^T dS), dO (row-wise for dP = dO V^T, transposed
// for dV^T += dO^T P), 64 rescaled logsumexps, 64 deltas.
// ---------------------------------------------------------------------------------------------------------
// WRITE_DS (regular lengths, no ALiBi): every 32-query x 32-key block of dS that a wave forms is also written to
// a.ds_blocks, in the wave's operand order, for fa_bwd_dq_from_ds.
template <bool BF16, int D, bool MASKED, int LAYOUT, bool ALIBI, bool DROPOUT, bool WRITE_DS = false>
__global__ void __launch_bounds__(kBwdWaves * 64, 2) fa_bwd_dkdv(const FaBwdArgs a)
{
    constexpr bool STRIDES = LAYOUT >= 1, GENERAL = LAYOUT == 2, ONE_ITEM = STRIDES && D == 128 && !(WRITE_DS && FA_DS_LOOP);
    static_assert(!WRITE_DS || LAYOUT <= 1 || (!ALIBI && !DROPOUT), "general lengths: dS blocks without ALiBi and dropout only");
    typedef Num<BF16> N;
    typedef TileReader<D> Reader;
    typedef TileLoader<D> Loader;
    constexpr int KS = Reader::KS, DB = Reader::DB, TILEB = Loader::TILEB, STAGEB = 2 * TILEB + 512, IPW = Loader::IPW;
    constexpr int NSTG = kBwdStages;                                  // LDS stages; pairs are requested NSTG - 1 ahead
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int S = a.S, Sk = GENERAL ? a.Sk : a.S, off = GENERAL ? a.Sk - a.S : 0;
    const int G = STRIDES ? a.H / a.Hk : 1;
    const int n_kblocks = (Sk + 255) / 256;
    // one K/V head per XCD at a time; key block 0 is seen by the most queries and goes first
    // (work items as in fa_bwd_dq; the list here is ascending in the key block, which is longest first under a
    // causal mask: key block 0 is seen by every query)
    const long long n_items = (long long)a.heads * n_kblocks;
    for (int pass = 0; !ONE_ITEM || pass < 1; ++pass) {       // (128-wide strided and general instantiations: exactly one item, no loop)
    const long long item = (long long)pass * gridDim.x + ((pass & 1) ? gridDim.x - 1 - blockIdx.x : blockIdx.x);
    if (item >= n_items) break;
    if (pass > 0) __syncthreads();
    int lane = ONE_ITEM ? (int)threadIdx.x & 63 : (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    if (!ONE_ITEM) asm volatile("" : "+v"(lane));
    const int half = lane >> 5, l32 = lane & 31;
    int bhk, kblock;
    fa_item_decode(item, a.heads, n_kblocks, 0, &bhk, &kblock);
    bhk += a.head0;
    const int b = bhk / a.Hk, hk = bhk - b * a.Hk;
    const int q_rs = STRIDES ? a.q.rs : D, g_rs = STRIDES ? a.dO_.rs : D, k_rs = STRIDES ? a.k.rs : D, v_rs = STRIDES ? a.v.rs : D;
    const uint16_t *Kh, *Vh;
    if (STRIDES) {
        Kh = head_ptr(a.K, a.k, b, hk); Vh = head_ptr(a.V, a.v, b, hk);
    } else {
        const size_t head_off = (size_t)bhk * S * D;
        Kh = a.K + head_off; Vh = a.V + head_off;
    }
    const int k0 = kblock * 256, kw = k0 + wave * 32;
    const bool active = kw < Sk;
    const int my_k = kw + l32;                     // this lane's key (masks, ALiBi)
    const int my_kc = active ? (GENERAL && my_k >= Sk ? Sk - 1 : my_k) : (GENERAL ? 0 : l32);     // row to load

    u32x4 kf[KS], vf[KS];           // K^T and V^T as B operands: lane = (key, head-dim slice)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        kf[s] = *reinterpret_cast<const u32x4 *>(Kh + (size_t)my_kc * k_rs + 16 * s + 8 * half);
        vf[s] = *reinterpret_cast<const u32x4 *>(Vh + (size_t)my_kc * v_rs + 16 * s + 8 * half);
    }
    const float c = a.scale * kLog2e;

    // the query tiles that see these keys: the query at index i (position i + off) sees key j iff
    // j - R - off <= i <= j + L - off: the forward bounds with the two sides exchanged and shifted
    const int Lq = a.R + off, Rq = a.L - off;
    int t0, t1, my_lo = 1, my_hi = 0;
    fa_tile_range(S, 64, Lq, Rq, k0, Sk - k0 < 256 ? Sk - k0 : 256, &t0, &t1);
    if (active) fa_tile_range(S, 64, Lq, Rq, kw, GENERAL && Sk - kw < 32 ? Sk - kw : 32, &my_lo, &my_hi);

    Reader rd; rd.init(lane, lds0);
    uint32_t stat_addr = lds0 + 2 * TILEB + 16 * half;       // this lane's logsumexp / delta words in the stage being read
    // dropout: 128 bytes per wave behind the ring, through which keep bits drawn with the query on the lane (one
    // Philox block covers sixteen keys of ONE query) reach the lanes that own the keys
    const uint32_t drop_lds = lds0 + NSTG * STAGEB + wave * 128;
    Loader ldq, ldg;
    if (!STRIDES || GENERAL) ldq.init(wave, lane, q_rs * 2);      // (general: only its ragged tiles go through these two)
    if (GENERAL) ldg.init(wave, lane, g_rs * 2);
    // strided layouts: where the walked query head starts (Q, dO, its rescaled logsumexps and deltas), formed when the
    // walk moves to the next head of the group and carried in eight scalar registers; the strides themselves are
    // read again at every fetch
    const uint16_t *walk_q = nullptr, *walk_g = nullptr;
    const float *walk_lse = nullptr, *walk_delta = nullptr;
    auto walk_head = [&](int g) __attribute__((always_inline)) {
        const FaBwdArgs &f = args_reloaded();
        const int h = hk * G + g;
        walk_q = head_ptr(f.Q, f.q, b, h); walk_g = head_ptr(f.dO, f.dO_, b, h);
        walk_lse = f.lse2 + ((size_t)b * f.H + h) * S; walk_delta = f.delta + ((size_t)b * f.H + h) * S;
    };
    // g: query head inside the group of this K/V head
    auto issue = [&](int g, int tile, int stage) __attribute__((always_inline)) {
        const uint32_t base = lds0 + stage * STAGEB;
        const int h = hk * G + g;
        const uint16_t *Qh, *dOh;
        const float *lse_h, *delta_h;
        if (STRIDES) {
            Qh = walk_q; dOh = walk_g; lse_h = walk_lse; delta_h = walk_delta;
        } else {
            Qh = a.Q + (size_t)bhk * S * D; dOh = a.dO + (size_t)bhk * S * D;
            lse_h = a.lse2 + ((size_t)b * a.H + h) * S; delta_h = a.delta + ((size_t)b * a.H + h) * S;
        }
        if (GENERAL && (tile + 1) * 64 > S) {
            const int valid = S - tile * 64;
            ldq.load_ragged(Qh + (size_t)tile * 64 * q_rs, base, valid, q_rs * 2);
            ldg.load_ragged(dOh + (size_t)tile * 64 * g_rs, base + TILEB, valid, g_rs * 2);
            int ln = lane;
            asm volatile("" : "+v"(ln));
            if (wave == 0) dma_4(lse_h + tile * 64, ln < valid ? ln : valid - 1, base + 2 * TILEB);
            if (wave == 1) dma_4(delta_h + tile * 64, ln < valid ? ln : valid - 1, base + 2 * TILEB + 256);
        } else if (STRIDES) {
            // (the lanes' source offsets are formed here, from the hardware's lane index and freshly loaded strides:
            // kept in registers from the top of the item they are spilled, and every reload in the tile loop waits
            // for all loads in flight)
            const FaBwdArgs &f = args_reloaded();
            int ln = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
            asm volatile("" : "+v"(ln));
            Loader lq, lg;
            lq.init(wave, ln, f.q.rs * 2);
            lg.init(wave, ln, f.dO_.rs * 2);
            lq.load(Qh + (size_t)tile * 64 * f.q.rs, base);
            lg.load(dOh + (size_t)tile * 64 * f.dO_.rs, base + TILEB);
            if (wave == 0) dma_4(lse_h + tile * 64, ln, base + 2 * TILEB);
            if (wave == 1) dma_4(delta_h + tile * 64, ln, base + 2 * TILEB + 256);
        } else {
            ldq.load(Qh + (size_t)tile * 64 * q_rs, base);
            ldq.load(dOh + (size_t)tile * 64 * g_rs, base + TILEB);
            if (wave == 0) dma_4(lse_h + tile * 64, lane, base + 2 * TILEB);
            if (wave == 1) dma_4(delta_h + tile * 64, lane, base + 2 * TILEB + 256);
        }
    };
    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) { dk[db] = zero16(); dv[db] = zero16(); }
    // WRITE_DS, head dimension 128: the kernel needs every register it can have (two waves per SIMD: 256), and a
    // value the compiler spills to scratch memory inside the tile loop comes back behind a wait for ALL loads and
    // stores in flight.  The last PARKED of the K^T and V^T fragments, which every half tile uses once, are kept in
    // LDS instead (32 bytes per lane and fragment pair, written once per work item) and read like any A operand.
    constexpr int PARKED = WRITE_DS && D == 128 ? (DROPOUT ? FA_PARK_DROP : ALIBI ? 2 : 1) : 0;
    constexpr uint32_t kParkPlane = 16u * kBwdWaves * 64u;
    const uint32_t park_lds = lds0 + NSTG * STAGEB + (DROPOUT ? kBwdWaves * 128 : 0);       // (behind the dropout words)
    auto parked = [&](int which, int s) __attribute__((always_inline)) {
        uint32_t ln = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        asm volatile("" : "+v"(ln));
        const uint32_t addr = park_lds + 16u * ((uint32_t)wave * 64u + ln) + kParkPlane * (uint32_t)(2 * (s - (KS - PARKED)) + which);
        return *(volatile __attribute__((address_space(3))) u32x4 *)(uintptr_t)addr;
    };

    // 32 queries (block qb of the tile in the stage being read) against this wave's 32 keys
    auto half_tile = [&](bool edge, float slope_l2, uint32_t bhq, int t, int qb) __attribute__((always_inline)) {
        constexpr int q_tile = 0, g_tile = TILEB;
        if (DROPOUT) {
            // lane (l32, half) draws for query 32*qb + l32 of the tile the sixteen keys 8*g + 4*half + e of this
            // wave's 32-key block and leaves them as a 16-bit mask (bit 4*g + e) in LDS word [half][l32]
            const DropWords dw = dropout_words(a.seed_lo, a.seed_hi, bhq, (uint32_t)(t * 64 + 32 * qb + l32 + off), (uint32_t)(2 * (kw >> 5) + half));
            uint32_t m = 0;
#pragma unroll
            for (int r = 0; r < 16; ++r) m |= dropout_keep_byte(dw, r, a.drop_threshold) ? (1u << r) : 0u;
            *(__attribute__((address_space(3))) uint16_t *)(drop_lds + (uint32_t)(half * 32 + l32) * 2u) = (uint16_t)m;
        }
        f32x16 sx = zero16();            // rows = queries, column (lane) = key
#pragma unroll
        for (int s = 0; s < KS; ++s) sx = N::mfma(rd.rows(q_tile, s, qb), s >= KS - PARKED ? parked(0, s) : kf[s], sx);      // S = Q K^T
        const int first = t * 64 + 32 * qb + 4 * half;                      // query of accumulator row 0 on this lane
        if (MASKED && edge) {            // wave-uniform; a masked score becomes -inf and its P exactly 0
            int hi = my_k + Rq, lo = my_k - Lq - first;                      // visible: lo <= 8*(r/4) + r%4 <= hi
            if (GENERAL && hi > S - 1) hi = S - 1;
            hi -= first;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (8 * (r >> 2) + (r & 3) > hi || 8 * (r >> 2) + (r & 3) < lo) sx[r] = -INFINITY;
        }
        // accumulator row r is query 32*qb + 8*(r/4) + 4*half + r%4 of the tile
        uint32_t keep = 0xffffu;         // bit r: the forward kept (query of row r, this lane's key)
        if (DROPOUT) {
            // this lane's key is key l32 of the block: drawn by the lanes of half (l32 / 4) % 2 as bit 4*(l32/8) + l32%4;
            // the four queries 8*g + 4*half + 0..3 sit in four consecutive 16-bit words
            const uint32_t src = drop_lds + (uint32_t)(((l32 >> 2) & 1) * 32 + 4 * half) * 2u, bit = (uint32_t)(4 * (l32 >> 3) + (l32 & 3));
            keep = 0;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const u32x2 w = *(const __attribute__((address_space(3))) u32x2 *)(src + 16u * g);
                const uint32_t w0 = w[0], w1 = w[1];
                keep |= ((w0 >> bit) & 1u) << (4 * g) | ((w0 >> (16 + bit)) & 1u) << (4 * g + 1) |
                        ((w1 >> bit) & 1u) << (4 * g + 2) | ((w1 >> (16 + bit)) & 1u) << (4 * g + 3);
            }
        }
        uint32_t pp[8];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const u32x4 lraw = lds_read_b128(stat_addr + (uint32_t)(32 * qb + 8 * g) * 4u);
            float p[4], pd[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = 4 * g + e;
                float x = __builtin_fmaf(sx[r], c, -as_f32(lraw[e]));
                if (ALIBI) x = __builtin_fmaf(-slope_l2, __builtin_fabsf((float)(first + 8 * g + e + off - my_k)), x);
                p[e] = __builtin_amdgcn_exp2f(x);
                sx[r] = p[e];                    // keep P in fp32 for dS
                pd[e] = DROPOUT ? (((keep >> r) & 1u) ? p[e] * a.drop_scale : 0.0f) : p[e];      // what multiplied V
            }
            pp[2 * g] = N::pack2(pd[0], pd[1]);
            pp[2 * g + 1] = N::pack2(pd[2], pd[3]);
        }
#pragma unroll
        for (int n = 0; n < 2 * DB; ++n) {                // dV^T += dO^T P
            const int h2 = n / DB, db = n % DB;
            const u32x4 bfrag = {pp[4 * h2], pp[4 * h2 + 1], pp[4 * h2 + 2], pp[4 * h2 + 3]};
            dv[db] = N::mfma(rd.transposed(g_tile, 2 * qb + h2, db), bfrag, dv[db]);
        }
        f32x16 dp = zero16();
#pragma unroll
        for (int s = 0; s < KS; ++s) dp = N::mfma(rd.rows(g_tile, s, qb), s >= KS - PARKED ? parked(1, s) : vf[s], dp);      // dP = dO V^T
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const u32x4 draw = lds_read_b128(stat_addr + 256u + (uint32_t)(32 * qb + 8 * g) * 4u);
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float dpr = dp[4 * g + e];
                if (DROPOUT) dpr = ((keep >> (4 * g + e)) & 1u) ? dpr * a.drop_scale : 0.0f;
                v[e] = sx[4 * g + e] * (dpr - as_f32(draw[e]));
            }
            pp[2 * g] = N::pack2(v[0], v[1]);     // now dS, same operand order
            pp[2 * g + 1] = N::pack2(v[2], v[3]);
        }
        if (WRITE_DS) {
            // Block (32-query block 2t + qb, this wave's 32-key block) of dS, 2 KiB, as the registers hold it: this
            // lane's key against the queries 8g + 4*half + 0..3, g = 0..3.  Two store instructions of 1 KiB each,
            // lane l writing bytes 16 l .. 16 l + 15 of its KiB: queries of g = 0, 1 in the first, g = 2, 3 in the second.
            // (bhq: the QUERY head, batch * H + head; the blocks of the query heads that share this K/V head are apart)
            const long long block = (long long)(bhq - (uint32_t)(a.head0 * G)) * fa_ds_blocks_per_head(S) + fa_ds_block_index(S, 2 * t + qb, kw >> 5);
            // (Inline assembly: the block's address stays in two scalar registers and the lane's offset in one
            // vector register that lives for these two instructions only -- as a 64-bit vector address it cost
            // the registers that made the compiler spill inside the tile loop, and every reload from scratch
            // memory there waits for all tile loads in flight.  Streaming stores: the blocks are read once, by
            // another kernel, and should not displace the walked tiles from L2.  The wait states cover the rule
            // that a store of more than 8 bytes must not be followed at once by a write of its data registers.)
            const uint64_t dst = (uint64_t)(reinterpret_cast<char *>(a.ds_blocks) + block * kDsBlockBytes);
            const uint64_t ub = ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(dst >> 32)) << 32) |
                                (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)dst);
            const uint32_t voff = 16u * __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
            u32x4 w0 = {pp[0], pp[1], pp[2], pp[3]}, w1 = {pp[4], pp[5], pp[6], pp[7]};
            // (general lengths: a lane whose key lies past the end has worked on a copy of the last key; what the
            // query-owning kernel multiplies with the padding rows of its last key tile must be zero)
            if (GENERAL && my_k >= Sk) { w0 = u32x4{0, 0, 0, 0}; w1 = u32x4{0, 0, 0, 0}; }
            asm volatile("global_store_dwordx4 %0, %1, %3 nt\n\tglobal_store_dwordx4 %0, %2, %3 offset:1024 nt\n\ts_nop 1"
                         :: "v"(voff), "v"(w0), "v"(w1), "s"(ub) : "memory");
        }
#pragma unroll
        for (int n = 0; n < 2 * DB; ++n) {                // dK^T += Q^T dS
            const int h2 = n / DB, db = n % DB;
            const u32x4 bfrag = {pp[4 * h2], pp[4 * h2 + 1], pp[4 * h2 + 2], pp[4 * h2 + 3]};
            dk[db] = N::mfma(rd.transposed(q_tile, 2 * qb + h2, db), bfrag, dk[db]);
        }
    };

    if (t0 <= t1) {
        // from the last query tile down to the diagonal: every workgroup of a head then starts on the same tile
        // and the ones that run together keep reading the same tiles out of L2; then the next head of the group
        // (head, tile) pairs are fetched two ahead, as in fa_bwd_dq
        int ig = 0, it = t1;                                    // the next pair to fetch
        auto issue_next = [&](int stage) __attribute__((always_inline)) {
            issue(ig, it, stage);
            if (--it < t0) {
                it = t1; ++ig;
                if (STRIDES && ig < G) walk_head(ig);
            }
        };
        if (STRIDES) walk_head(0);
        issue_next(0);
        if (ig < G) issue_next(1);
        wait_vm<0>();
#pragma unroll
        for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(kf[s]), "+v"(vf[s]));
        if (PARKED > 0) {           // from here on the last fragments live in LDS, and their registers are free
            // (one plane of 16 bytes per thread for every parked fragment: consecutive lanes, consecutive 16 bytes)
            const uint32_t slot = park_lds + 16u * (uint32_t)(wave * 64 + lane);
#pragma unroll
            for (int i = 0; i < PARKED; ++i) {
                *(__attribute__((address_space(3))) u32x4 *)(uintptr_t)(slot + kParkPlane * (2 * i)) = kf[KS - PARKED + i];
                *(__attribute__((address_space(3))) u32x4 *)(uintptr_t)(slot + kParkPlane * (2 * i + 1)) = vf[KS - PARKED + i];
            }
        }
        int stage = 0;
        // WRITE_DS: the dS stores this wave made in the last two iterations, and the pairs still to come.  The next
        // pair is then requested in front of an iteration's work instead of behind it.
        int st1 = 0, st2 = 0, pairs_left = G * (t1 - t0 + 1);
        constexpr bool TOP = WRITE_DS;
        for (int g = 0; g < G; ++g) {
            float slope_l2 = 0.0f;
            if (ALIBI) slope_l2 = a.alibi[hk * G + g] * kLog2e;
            for (int t = t1; t >= t0; --t) {
                const int next = stage == NSTG - 1 ? 0 : stage + 1, prev = stage == 0 ? NSTG - 1 : stage - 1;
                const bool more = t - 1 >= t0 || g + 1 < G;
                --pairs_left;
                if (WRITE_DS) {
                    // This pair has landed when at most what was issued behind it is outstanding (memory operations
                    // complete in the order they were issued): the loads of the pairs requested since, and the dS
                    // stores made since.  Requests at the top of an iteration put a pair's loads in front of that
                    // iteration's stores, so a store that takes long to be acknowledged holds up no load needed now.
                    const int loads = wave < 2 ? 2 * IPW + 1 : 2 * IPW;     // waves 0 and 1 also fetch lse / delta
                    wait_vm_upto((pairs_left > 0 ? loads : 0) + st1 + st2);
                } else if (more) {                              // this pair has landed, the next may still be in flight
                    if (wave < 2) wait_vm<2 * IPW + 1>(); else wait_vm<2 * IPW>();     // waves 0 and 1 also fetch lse / delta
                } else wait_vm<0>();
                phase_barrier();
                if (TOP && ig < G) issue_next(prev);
                st2 = st1;
                st1 = (WRITE_DS && my_lo <= t && t <= my_hi) ? 4 : 0;
                if (my_lo <= t && t <= my_hi) {
                    const bool edge = MASKED && (fa_tile_class(64, Lq, Rq, kw, 32, t) == 1 || (GENERAL && (t + 1) * 64 > S));
                    const uint32_t bhq = (uint32_t)(b * a.H + hk * G + g);        // the head the forward keyed its dropout on
                    half_tile(edge, slope_l2, bhq, t, 0);
                    half_tile(edge, slope_l2, bhq, t, 1);
                }
                if (!TOP && ig < G) issue_next(prev);
                rd.advance(next == 0 ? -(NSTG - 1) * STAGEB : STAGEB);
                stat_addr += next == 0 ? -(NSTG - 1) * STAGEB : STAGEB;
                stage = next;
            }
        }
    }
    // (the lane's row and column offset are derived again here, from the hardware's lane index and tied to this
    // place: taken from the values computed at the top, the compiler forms the store addresses there and keeps
    // them in registers, or in scratch memory, through the whole loop)
    int lane_e = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(lane_e));
    const int key_e = kw + (lane_e & 31), half_e = lane_e >> 5;
    if (active && key_e < Sk) {
        uint16_t *dKh, *dVh;
        int dk_rs = D, dv_rs = D;
        if (STRIDES) {
            const FaBwdArgs &f = args_reloaded();
            dKh = head_ptr(f.dK, f.dk, b, hk); dVh = head_ptr(f.dV, f.dv, b, hk);
            dk_rs = f.dk.rs; dv_rs = f.dv.rs;
        } else {
            dKh = a.dK + (size_t)bhk * S * D; dVh = a.dV + (size_t)bhk * S * D;
        }
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 wk, wv;
                wk[0] = N::pack2(dk[db][4 * g] * a.scale, dk[db][4 * g + 1] * a.scale);
                wk[1] = N::pack2(dk[db][4 * g + 2] * a.scale, dk[db][4 * g + 3] * a.scale);
                wv[0] = N::pack2(dv[db][4 * g], dv[db][4 * g + 1]);
                wv[1] = N::pack2(dv[db][4 * g + 2], dv[db][4 * g + 3]);
                *reinterpret_cast<u32x2 *>(dKh + (size_t)key_e * dk_rs + 32 * db + 8 * g + 4 * half_e) = wk;
                *reinterpret_cast<u32x2 *>(dVh + (size_t)key_e * dv_rs + 32 * db + 8 * g + 4 * half_e) = wv;
            }
    }
    }   // next work item
}

// ---------------------------------------------------------------------------------------------------------
// The five-product form (regular lengths in the reference's or a strided layout, no ALiBi).  fa_bwd_dq above and fa_bwd_dkdv each recompute S and dP: seven
// products for five.  Here fa_bwd_dkdv, which has every dS block in registers as the operand of dK += dS^T Q,
// also writes it out (WRITE_DS), and dQ = scale * dS K is one product over those blocks: every output element
// still has exactly one writer and the same inputs give the same bits.  The price is S*S_kv storage-type elements
// per head written once and read once, so this kernel is bound by HBM bandwidth, not by the matrix cores.
//
// fa_bwd_prepare: delta_i = sum_t dO_it O_it and the logsumexp in exp2 units, which fa_bwd_dkdv fetches per
// query tile (fa_bwd_dq writes them in the seven-product form).
// ---------------------------------------------------------------------------------------------------------
template <bool BF16, int D, bool STRIDED>
__global__ void __launch_bounds__(256) fa_bwd_prepare(const FaBwdArgs a)
{
    constexpr int TPR = D / 8;                    // threads per row, 16 bytes each
    const long long row = (long long)blockIdx.x * (256 / TPR) + threadIdx.x / TPR;
    const long long n_rows = (long long)a.B * a.H * a.S;
    const bool live = row < n_rows;
    const long long r = live ? row : n_rows - 1;
    const int c = (threadIdx.x % TPR) * 8;
    const uint16_t *o_row = a.O + r * D, *g_row = a.dO + r * D;
    if (STRIDED) {                                // row r of the [B,H,S] order, wherever the tensors keep it
        const long long bh = r / a.S;
        const int i = (int)(r - bh * a.S), b = (int)(bh / a.H), h = (int)(bh - (long long)b * a.H);
        o_row = head_ptr(a.O, a.o, b, h) + (long long)i * a.o.rs;
        g_row = head_ptr(a.dO, a.dO_, b, h) + (long long)i * a.dO_.rs;
    }
    const u32x4 o = *reinterpret_cast<const u32x4 *>(o_row + c);
    const u32x4 g = *reinterpret_cast<const u32x4 *>(g_row + c);
    float sum = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t ow = o[w], gw = g[w];
        sum += storage_to_f32<BF16>((uint16_t)(ow & 0xffffu)) * storage_to_f32<BF16>((uint16_t)(gw & 0xffffu));
        sum += storage_to_f32<BF16>((uint16_t)(ow >> 16)) * storage_to_f32<BF16>((uint16_t)(gw >> 16));
    }
#pragma unroll
    for (int m = 1; m < TPR; m <<= 1) sum += __shfl_xor(sum, m);
    if (live && threadIdx.x % TPR == 0) {
        a.delta[row] = sum;
        const float l = a.lse[row];
        a.lse2[row] = l == -INFINITY ? INFINITY : l * kLog2e;
    }
}

// dQ^T += K^T dS^T over the dS blocks fa_bwd_dkdv<WRITE_DS> wrote.  A workgroup owns 256 queries (8 waves x one
// 32-query block, lane = query) and walks the key tiles of its visible range.  LDS stage: the K tile (read
// transposed, as in fa_bwd_dq) and, per wave, the two 2 KiB dS blocks of its query block against the tile's keys,
// fetched by that wave alone.  A block comes in as it lies in memory except that the 64-byte groups of four keys
// are XOR-permuted among the four 512-byte planes, so that the transposing read of a half-wave -- four keys, all
// 32 queries, i.e. one group in each plane -- touches every LDS bank once.
template <bool BF16, int D, bool MASKED, int LAYOUT>
__global__ void __launch_bounds__(kBwdWaves * 64, 2) fa_bwd_dq_from_ds(const FaBwdArgs a)
{
    constexpr bool STRIDED = LAYOUT >= 1, GENERAL = LAYOUT == 2;      // (general: any length S = S_kv)
    typedef Num<BF16> N;
    typedef TileReader<D> Reader;
    typedef TileLoader<D> Loader;
    constexpr int DB = Reader::DB, TILEB = Loader::TILEB, IPW = Loader::IPW;
    constexpr int WAVE_DS = 2 * kDsBlockBytes;                 // a wave's two blocks of a key tile
    constexpr int STAGEB = TILEB + kBwdWaves * WAVE_DS;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int S = a.S;
    const int n_qblocks = (S + 255) / 256;
    const int group = STRIDED ? a.H / a.Hk : 1, heads_q = a.heads * group, head0_q = a.head0 * group;
    const long long n_items = (long long)heads_q * n_qblocks;
    for (int pass = 0;; ++pass) {
    const long long item = (long long)pass * gridDim.x + ((pass & 1) ? gridDim.x - 1 - blockIdx.x : blockIdx.x);
    if (item >= n_items) break;
    if (pass > 0) __syncthreads();          // (the LDS stages: other waves may still be reading the last tile)
    int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(lane));
    const int half = lane >> 5, l32 = lane & 31, l16 = lane & 15;
    int bh, qblock;
    fa_item_decode(item, heads_q, n_qblocks, MASKED ? 1 : 0, &bh, &qblock);
    bh += head0_q;
    const uint16_t *Kh = a.K + (size_t)bh * S * D;
    uint16_t *dQh = a.dQ + (size_t)bh * S * D;
    int k_rs = D, dq_rs = D;
    if (STRIDED) {                                 // (bh counts query heads; the K/V head of query head h is h / (H / Hk))
        const int b = bh / a.H, h = bh - b * a.H;
        Kh = head_ptr(a.K, a.k, b, h / group);
        dQh = head_ptr(a.dQ, a.dq, b, h);
        k_rs = a.k.rs; dq_rs = a.dq.rs;
    }
    const int q0 = qblock * 256, qw = q0 + wave * 32;
    const bool active = qw < S;                    // the last block may own fewer than 256 rows
    int t0, t1, my_lo = 1, my_hi = 0;
    fa_tile_range(S, 64, a.L, a.R, q0, S - q0 < 256 ? S - q0 : 256, &t0, &t1);
    if (active) fa_tile_range(S, 64, a.L, a.R, qw, GENERAL && S - qw < 32 ? S - qw : 32, &my_lo, &my_hi);
    // this head's dS blocks; this wave reads those of query block qw / 32
    const char *ds_head = reinterpret_cast<const char *>(a.ds_blocks) + (long long)(bh - head0_q) * fa_ds_blocks_per_head(S) * kDsBlockBytes;
    const int my_qb = active ? qw >> 5 : 0;

    Reader rd; rd.init(lane, lds0);
    Loader ldk; ldk.init(wave, lane, k_rs * 2);
    // Source of the 16 bytes lane l brings in with instruction w (0, 1) of a block: LDS slot 64 w + l of the block
    // = plane p = 2 w + l / 32, position l % 32; that position holds key ((l % 32 / 4) ^ p) * 4 + l % 4, which lies
    // in memory at 1 KiB * w + 512 * (l / 32) + 16 * key.
    uint32_t ds_src[2];
#pragma unroll
    for (int w = 0; w < 2; ++w) {
        const int p = 2 * w + half, key = ((((l32 >> 2) ^ p) & 7) << 2) | (l32 & 3);
        ds_src[w] = (uint32_t)(1024 * w + 512 * half + 16 * key);
    }
    // Transposing read of a B operand (lane = query l32, keys 16 t2 + 4 half + {0..3} and + 8 of a block): the lane
    // addresses the 8 bytes that hold queries 16 (l32 / 16) + 4 (l16 % 4) .. + 3 of key 16 t2 + 8 hi + 4 half + l16 / 4.
    // Those four queries are quad 4 (l32 / 16) + l16 % 4 = 2 g + h of the block, written by fa_bwd_dkdv's lane
    // (key, half h) as its g-th pair of words: plane p = 2 (g / 2) + h, 16-byte slot of the key, byte 8 (g % 2).
    uint32_t ds_rd[2];
    {
        const int quad = 4 * (l32 >> 4) + (l16 & 3), g = quad >> 1, hq = quad & 1;
        const int p = 2 * (g >> 1) + hq;
#pragma unroll
        for (int hi = 0; hi < 2; ++hi)
            ds_rd[hi] = lds0 + TILEB + wave * WAVE_DS +
                        (uint32_t)(512 * p + ((((2 * hi + half) ^ p) & 3) << 6) + 16 * (l16 >> 2) + 8 * (g & 1));
    }
    auto issue = [&](int tile, int stage) __attribute__((always_inline)) {
        const uint32_t base = lds0 + stage * STAGEB;
        if (GENERAL && (tile + 1) * 64 > S) ldk.load_ragged(Kh + (size_t)tile * 64 * k_rs, base, S - tile * 64, k_rs * 2);
        else ldk.load(Kh + (size_t)tile * 64 * k_rs, base);
        if (my_lo <= tile && tile <= my_hi) {
            const char *src = ds_head + fa_ds_block_index(S, my_qb, 2 * tile) * kDsBlockBytes;      // (and its neighbour 2 tile + 1)
            const uint32_t dst = base + TILEB + wave * WAVE_DS;
#pragma unroll
            for (int n = 0; n < 4; ++n)         // block 2 tile (n = 0, 1), block 2 tile + 1 (n = 2, 3)
                dma_16_stream(src, (uint32_t)((n >> 1) * kDsBlockBytes) + ds_src[n & 1], dst + n * 1024);
        }
    };
    // the blocks fa_bwd_dkdv wrote: its wave with the 32 keys from `key0` on visits the query tiles of this range
    auto block_written = [&](int key0) __attribute__((always_inline)) {
        if (GENERAL && key0 >= S) return false;          // (a wave of the key-owning kernel without any key)
        int lo, hi;
        fa_tile_range(S, 64, a.R, a.L, key0, GENERAL && S - key0 < 32 ? S - key0 : 32, &lo, &hi);
        return lo <= (qw >> 6) && (qw >> 6) <= hi;
    };

    f32x16 dq[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db) dq[db] = zero16();

    if (t0 <= t1) {
        issue(t0, 0);
        if (t0 + 1 <= t1) issue(t0 + 1, 1);
        wait_vm<0>();
        int stage = 0;
        for (int t = t0; t <= t1; ++t) {
            const int next = stage == kBwdStages - 1 ? 0 : stage + 1;
            if (t + 1 <= t1) {              // tile t has landed, tile t+1 may still be in flight
                if (my_lo <= t + 1 && t + 1 <= my_hi) wait_vm<IPW + 4>(); else wait_vm<IPW>();
            } else wait_vm<0>();
            phase_barrier();
            if (my_lo <= t && t <= my_hi) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb) {
                    if ((MASKED || GENERAL) && !block_written(64 * t + 32 * kb)) continue;       // wave-uniform
#pragma unroll
                    for (int t2 = 0; t2 < 2; ++t2) {
                        const u32x2 lo = lds_read_tr(ds_rd[0] + (uint32_t)(kb * kDsBlockBytes + 256 * t2));
                        const u32x2 hi = lds_read_tr(ds_rd[1] + (uint32_t)(kb * kDsBlockBytes + 256 * t2));
                        const u32x4 bfrag = {lo[0], lo[1], hi[0], hi[1]};
#pragma unroll
                        for (int db = 0; db < DB; ++db) dq[db] = N::mfma(rd.transposed(0, 2 * kb + t2, db), bfrag, dq[db]);
                    }
                }
            }
            if (t + 2 <= t1) issue(t + 2, next == kBwdStages - 1 ? 0 : next + 1);
            const int delta = next == 0 ? -(kBwdStages - 1) * STAGEB : STAGEB;
            rd.advance(delta);
            ds_rd[0] += delta; ds_rd[1] += delta;
            stage = next;
        }
    }
    if (active && (!GENERAL || qw + l32 < S)) {
        const int my_q = qw + l32;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                u32x2 w;
                w[0] = N::pack2(dq[db][4 * g] * a.scale, dq[db][4 * g + 1] * a.scale);
                w[1] = N::pack2(dq[db][4 * g + 2] * a.scale, dq[db][4 * g + 3] * a.scale);
                *reinterpret_cast<u32x2 *>(dQh + (size_t)my_q * dq_rs + 32 * db + 8 * g + 4 * half) = w;
            }
    }
    }   // next work item
}

template <bool BF16, int D, bool MASKED, int LAYOUT, bool ALIBI, bool DROPOUT>
hipError_t launch_bwd(const FaBwdArgs &a_in, int compute_units, hipStream_t stream, bool configure_only = false)
{
    constexpr int TILEB = 64 * D * 2;
    FaBwdArgs a = a_in;
    const int all_heads = a.B * a.Hk, group = a.Hk > 0 ? a.H / a.Hk : 1;
    a.head0 = 0;
    a.heads = all_heads;
    const int smem_dq = kBwdStages * 2 * TILEB, smem_dkdv = kBwdStages * (2 * TILEB + 512) + (DROPOUT ? kBwdWaves * 128 : 0);
    const int smem_dkdv_ds = smem_dkdv + (D == 128 ? (DROPOUT ? FA_PARK_DROP : ALIBI ? 2 : 1) * 32 * kBwdWaves * 64 : 0);      // + the parked fragments
    auto kq = fa_bwd_dq<BF16, D, MASKED, LAYOUT, ALIBI, DROPOUT>;
    auto kkv = fa_bwd_dkdv<BF16, D, MASKED, LAYOUT, ALIBI, DROPOUT>;
    // the five-product form: regular lengths (the reference's layout or a strided one) with dropout or ALiBi, any
    // length S = S_kv without them
    constexpr bool FIVE = LAYOUT <= 1 || (!ALIBI && !DROPOUT);
    constexpr int FL = FIVE ? LAYOUT : 0;
    const int smem_dq_ds = kBwdStages * (TILEB + kBwdWaves * 2 * kDsBlockBytes);
    // the LDS opt-in is per (instantiation, device) and is made once, not on every launch
    static std::atomic<unsigned long long> configured{0ull};
    const unsigned long long dev_bit = 1ull << fa_launch_device();
    if (!(configured.load(std::memory_order_relaxed) & dev_bit)) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kq), hipFuncAttributeMaxDynamicSharedMemorySize, smem_dq);
        if (e != hipSuccess) return e;
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(kkv), hipFuncAttributeMaxDynamicSharedMemorySize, smem_dkdv);
        if (e != hipSuccess) return e;
        if constexpr (FIVE) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(fa_bwd_dkdv<BF16, D, MASKED, FL, ALIBI, DROPOUT, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem_dkdv_ds);
            if (e != hipSuccess) return e;
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(fa_bwd_dq_from_ds<BF16, D, MASKED, FL>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, smem_dq_ds);
            if (e != hipSuccess) return e;
        }
        configured.fetch_or(dev_bit, std::memory_order_relaxed);
    }
    if (configure_only) return hipSuccess;     // (fa_init: the opt-in alone, so that no launch inside a stream capture makes it)
    // Masked problems with between one and sixteen items per compute unit: a resident grid (one workgroup per CU,
    // 8 waves at two per SIMD) walks the list as a snake, which pairs every long item with a short one; otherwise
    // one workgroup per item, handed out by the hardware as CUs free up.  Causal fp16, snake against dispatch:
    // B1 H32 S4096 D128 477 against 639 us, B1 H64 S2048 D128 273 against 370, B4 H16 S2048 D64 160 against 221,
    // B8 H32 S1024 D64 194 against 237, c3's shape 3.59 against 3.64 ms; without a mask (items all alike) the
    // hardware's order is 1-7 % ahead.
    // (a window of at most half the length leaves the items alike too: c4's shape 1.14 ms in the hardware's order,
    // 1.16 as a snake)
    const unsigned resident = (unsigned)compute_units;
    // (the general instantiations always carry the mask code: without a bound on either side, L = R = S + S_kv, their
    // items are alike as well)
    const long long unbounded = (long long)a.S + a.Sk;
    // (The 128-wide strided and general instantiations are launched one workgroup per item only: with the item loop
    // around them they spill ten times as much, and a reload inside the tile loop waits for every tile load in
    // flight: c3's shape stored [B,S,H,D] 4.1 ms against 3.8.  The 64-wide ones have the registers for the loop.)
    // (The kernels of the five-product form have the loop in every layout: the key-owning one keeps K^T / V^T
    // fragments in LDS and compiles with it without spilling, or with 12 bytes outside the tile loop.)
    const bool uneven_items = MASKED && (a.L < unbounded || a.R < unbounded) && 2LL * a.L > (long long)a.S;
    const bool uneven = (LAYOUT == 0 || D == 64) && uneven_items;
    auto grid_if = [&](bool snake, long long items) {
        const unsigned g = (unsigned)items;
        return (snake && g > resident && g < 16u * resident) ? resident : g;
    };
    auto grid_for = [&](long long items) { return grid_if(uneven, items); };
    if constexpr (FIVE) {
        if (a.ds_blocks != nullptr) {
            // delta and the rescaled logsumexp, for all heads at once; then, for as many heads at a time as the
            // workspace holds dS blocks for: dK, dV and the dS blocks; dQ from the blocks
            constexpr int rows_per_block = 256 / (D / 8);
            const long long n_rows = (long long)a.B * a.H * a.S;
            hipLaunchKernelGGL((fa_bwd_prepare<BF16, D, FL >= 1>), dim3((unsigned)((n_rows + rows_per_block - 1) / rows_per_block)), dim3(256), 0, stream, a);
            const int chunk = a.ds_heads > 0 && a.ds_heads < all_heads ? a.ds_heads : all_heads;
            for (int h0 = 0; h0 < all_heads; h0 += chunk) {
                a.head0 = h0;
                a.heads = all_heads - h0 < chunk ? all_heads - h0 : chunk;
                const unsigned launch_k = grid_if(FA_DS_LOOP ? uneven_items : uneven, (long long)a.heads * ((a.Sk + 255) / 256));
                const unsigned launch_q = grid_if(uneven_items, (long long)a.heads * group * ((a.S + 255) / 256));
                hipLaunchKernelGGL((fa_bwd_dkdv<BF16, D, MASKED, FL, ALIBI, DROPOUT, true>), dim3(launch_k), dim3(kBwdWaves * 64), smem_dkdv_ds, stream, a);
                hipLaunchKernelGGL((fa_bwd_dq_from_ds<BF16, D, MASKED, FL>), dim3(launch_q), dim3(kBwdWaves * 64), smem_dq_ds, stream, a);
            }
            return hipGetLastError();
        }
    }
    const unsigned launch_q = grid_for((long long)a.B * a.H * ((a.S + 255) / 256));
    const unsigned launch_k = grid_for((long long)a.B * a.Hk * ((a.Sk + 255) / 256));
    hipLaunchKernelGGL(kq, dim3(launch_q), dim3(kBwdWaves * 64), smem_dq, stream, a);
    hipLaunchKernelGGL(kkv, dim3(launch_k), dim3(kBwdWaves * 64), smem_dkdv, stream, a);
    return hipGetLastError();
}

}  // namespace

#endif
