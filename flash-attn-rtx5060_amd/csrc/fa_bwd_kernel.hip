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
// Three kernels: fa_bwd_delta (one row per thread), fa_bwd_dq (a workgroup owns 128 queries and walks the key
// tiles) and fa_bwd_dkdv (a workgroup owns 128 keys and walks the query tiles); no atomics, every output
// element has one writer.  Both walkers use the building blocks of the forward kernel: 32x32x16 MFMA with the
// thing a wave owns on the lane (query in fa_bwd_dq, key in fa_bwd_dkdv), so that the owner's operands are B
// operands loaded once into registers, the walked tiles are A operands streamed through LDS by direct
// global->LDS loads, and an accumulator tile is already laid out as the B operand of the next product.
// A walked tile that is needed both row-wise (ds_read_b128) and transposed (ds_read_b64_tr_b16) is put into
// LDS twice, once in each of the two bank-conflict-free swizzles.
#include "fa_fwd_kernel_impl.h"
#include "fa_bwd_args.h"

namespace {

constexpr int kBwdWaves = 4;            // 4 waves x 32 owned rows = 128 rows per workgroup, one wave per SIMD
constexpr float kLog2e = 1.44269504088896340736f;

// Takes the word by value on purpose: __builtin_bit_cast applied directly to an element of a vector
// (`__builtin_bit_cast(float, v[e])`) reads element 0 whatever e is with this compiler.
__device__ __forceinline__ float as_f32(uint32_t w) { return __builtin_bit_cast(float, w); }

// per-lane LDS offsets of the two read patterns, relative to a tile's base (same formulas as the forward kernel)
template <int D> struct TileReader {
    static constexpr int CPR = D / 8, ROWB = D * 2, KS = D / 16, DB = D / 32;
    uint32_t row_off[KS];       // ds_read_b128: A operand rows = tile rows, k = 16 head-dim values of slice s
    uint32_t tr_off[DB];        // ds_read_b64_tr_b16: A operand rows = head dim (block db), k = 16 tile rows
    __device__ __forceinline__ void init(int lane)
    {
        const int half = lane >> 5, l32 = lane & 31, l16 = lane & 15;
#pragma unroll
        for (int s = 0; s < KS; ++s) row_off[s] = (uint32_t)(l32 * ROWB + (((2 * s + half) ^ k_swz<CPR>(l32)) << 4));
        const int row0 = 4 * half + (l16 >> 2), dq = l32 >> 4, c4 = l16 & 3;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
            const int c = 4 * db + 2 * dq + (c4 >> 1);
            tr_off[db] = (uint32_t)(row0 * ROWB + ((c ^ v_swz<CPR>(row0)) << 4) + ((c4 & 1) << 3));
        }
    }
    // fragment n of the row-wise pattern: head-dim slice n >> 1, 32-row block n & 1 of a tile stored with k_swz
    __device__ __forceinline__ u32x4 rows(uint32_t tile, int n) const { return lds_read_b128(tile + row_off[n >> 1] + (n & 1) * 32 * ROWB); }
    // fragment n of the transposed pattern: 16-row slice n / DB, head-dim block n % DB of a tile stored with v_swz
    __device__ __forceinline__ u32x4 transposed(uint32_t tile, int n) const
    {
        const int t2 = n / DB, db = n % DB;
        const u32x2 lo = lds_read_tr(tile + tr_off[db] + (16 * t2) * ROWB);
        const u32x2 hi = lds_read_tr(tile + tr_off[db] + (16 * t2 + 8) * ROWB);
        return u32x4{lo[0], lo[1], hi[0], hi[1]};
    }
};

// one 64-row tile global -> LDS: wave w issues instructions w, w+4, ... ; `rowwise` picks the swizzle
template <int D> struct TileLoader {
    static constexpr int CPR = D / 8, ROWB = D * 2, TILEB = 64 * ROWB, IPW = TILEB / 1024 / kBwdWaves;
    uint32_t g_row[IPW], g_tr[IPW];
    int wave;
    __device__ __forceinline__ void init(int wave_, int lane)
    {
        wave = wave_;
#pragma unroll
        for (int i = 0; i < IPW; ++i) {
            const int P = (i * kBwdWaves + wave) * 64 + lane, row = P / CPR, pos = P % CPR;
            g_row[i] = (uint32_t)(row * ROWB + ((pos ^ k_swz<CPR>(row)) << 4));
            g_tr[i] = (uint32_t)(row * ROWB + ((pos ^ v_swz<CPR>(row)) << 4));
        }
    }
    __device__ __forceinline__ void load(const uint16_t *tile_src, uint32_t lds_tile, bool rowwise) const
    {
#pragma unroll
        for (int i = 0; i < IPW; ++i)
            dma_16(reinterpret_cast<const char *>(tile_src), rowwise ? g_row[i] : g_tr[i], lds_tile + (i * kBwdWaves + wave) * 1024);
    }
};

// 256 bytes (64 floats) global -> LDS in one wave instruction: lane l copies 4 bytes to LDS byte lds + 4*l
__device__ __forceinline__ void dma_4(const float *src, int lane, uint32_t lds)
{
    const uint64_t b = (uint64_t)src;
    const uint32_t b_hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(b >> 32));
    const uint32_t b_lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)b);
    const uint64_t ub = ((uint64_t)b_hi << 32) | (uint64_t)b_lo;
    const uint32_t voff = (uint32_t)lane * 4u;
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds)), "v"(voff), "s"(ub) : "memory");
}

// ---------------------------------------------------------------------------------------------------------
// delta_i = sum_t dO_it * O_it, fp32 [B,H,S]
// ---------------------------------------------------------------------------------------------------------
template <bool BF16, int D>
__global__ void __launch_bounds__(256) fa_bwd_delta(const FaBwdArgs a)
{
    const long long row = (long long)blockIdx.x * 256 + threadIdx.x;
    if (row >= (long long)a.BH * a.S) return;
    const u32x4 *o = reinterpret_cast<const u32x4 *>(a.O + (size_t)row * D);
    const u32x4 *g = reinterpret_cast<const u32x4 *>(a.dO + (size_t)row * D);
    float sum = 0.0f;
#pragma unroll
    for (int c = 0; c < D / 8; ++c) {
        const u32x4 x = o[c], y = g[c];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            sum += storage_to_f32<BF16>((uint16_t)(x[w] & 0xffffu)) * storage_to_f32<BF16>((uint16_t)(y[w] & 0xffffu));
            sum += storage_to_f32<BF16>((uint16_t)(x[w] >> 16)) * storage_to_f32<BF16>((uint16_t)(y[w] >> 16));
        }
    }
    a.delta[row] = sum;
}

// ---------------------------------------------------------------------------------------------------------
// dQ: a workgroup owns 128 queries (lane = query), walks the key tiles of its visible range.
// LDS stage: K row-wise, K transposed-pattern, V row-wise.
// ---------------------------------------------------------------------------------------------------------
template <bool BF16, int D, bool MASKED>
__global__ void __launch_bounds__(kBwdWaves * 64, 1) fa_bwd_dq(const FaBwdArgs a)
{
    typedef Num<BF16> N;
    typedef TileReader<D> Reader;
    typedef TileLoader<D> Loader;
    constexpr int KS = Reader::KS, DB = Reader::DB, TILEB = Loader::TILEB, STAGEB = 3 * TILEB, IPW = Loader::IPW;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int S = a.S;
    const int n_qblocks = S / 128;
    // one head per XCD at a time, long blocks first: the workgroups that share a head's K and V share an L2
    int bh, qblock;
    fa_item_decode((long long)blockIdx.x, a.BH, n_qblocks, MASKED ? 1 : 0, &bh, &qblock);
    const size_t head_off = (size_t)bh * S * D;
    const uint16_t *Qh = a.Q + head_off, *Kh = a.K + head_off, *Vh = a.V + head_off, *dOh = a.dO + head_off;
    const int q0 = qblock * 128, qw = q0 + wave * 32, my_q = qw + l32;

    u32x4 qf[KS], gf[KS];           // Q^T and dO^T as B operands: lane = (query, head-dim slice 8*half..+7 of each 16)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        qf[s] = *reinterpret_cast<const u32x4 *>(Qh + (size_t)my_q * D + 16 * s + 8 * half);
        gf[s] = *reinterpret_cast<const u32x4 *>(dOh + (size_t)my_q * D + 16 * s + 8 * half);
    }
    float lse_l2 = a.lse[(size_t)bh * S + my_q] * kLog2e;
    float delta = a.delta[(size_t)bh * S + my_q];
    const float c = a.scale * kLog2e;

    int t0, t1, my_lo, my_hi;
    fa_tile_range(S, 64, a.L, a.R, q0, 128, &t0, &t1);
    fa_tile_range(S, 64, a.L, a.R, qw, 32, &my_lo, &my_hi);

    Reader rd; rd.init(lane);
    Loader ld; ld.init(wave, lane);
    auto issue = [&](int tile, int stage) __attribute__((always_inline)) {
        const uint32_t base = lds0 + stage * STAGEB;
        ld.load(Kh + (size_t)tile * 64 * D, base, true);
        ld.load(Kh + (size_t)tile * 64 * D, base + TILEB, false);
        ld.load(Vh + (size_t)tile * 64 * D, base + 2 * TILEB, true);
    };

    f32x16 dq[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) dq[db][r] = 0.0f;

    if (t0 <= t1) {
        issue(t0, 0);
        wait_vm<0>();
        // the owner's operands have landed too: say so, or the compiler waits for them inside the loop, where
        // its wait would also cover the asynchronous tile loads
#pragma unroll
        for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(qf[s]), "+v"(gf[s]));
        asm volatile("" : "+v"(lse_l2), "+v"(delta));
        for (int t = t0; t <= t1; ++t) {
            const int stage = (t - t0) & 1;
            if (t + 1 <= t1) { issue(t + 1, stage ^ 1); wait_vm<3 * IPW>(); }
            else wait_vm<0>();
            phase_barrier();                                    // tile t is in LDS for everyone
            if (my_lo <= t && t <= my_hi) {
                const uint32_t k_rows = lds0 + stage * STAGEB, k_tr = k_rows + TILEB, v_rows = k_rows + 2 * TILEB;
                f32x16 sx[2], dp[2];
#pragma unroll
                for (int r = 0; r < 16; ++r) { sx[0][r] = 0.0f; sx[1][r] = 0.0f; dp[0][r] = 0.0f; dp[1][r] = 0.0f; }
#pragma unroll
                for (int n = 0; n < 2 * KS; ++n) sx[n & 1] = N::mfma(rd.rows(k_rows, n), qf[n >> 1], sx[n & 1]);     // S^T = K Q^T
#pragma unroll
                for (int n = 0; n < 2 * KS; ++n) dp[n & 1] = N::mfma(rd.rows(v_rows, n), gf[n >> 1], dp[n & 1]);     // dP^T = V dO^T
                const bool edge = MASKED && fa_tile_class(64, a.L, a.R, qw, 32, t) == 1;
                uint32_t ds[16];                                 // dS^T in B-operand order: [0..7] keys 0..31, [8..15] keys 32..63
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int i = 0; i < 8; ++i) {
                        float v[2];
#pragma unroll
                        for (int e = 0; e < 2; ++e) {
                            const int r = 2 * i + e;
                            const int j = t * 64 + 32 * kb + 8 * (r >> 2) + 4 * half + (r & 3);
                            float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sx[kb][r], c, -lse_l2));
                            if (edge && (j > my_q + a.R || j < my_q - a.L)) p = 0.0f;
                            v[e] = p * (dp[kb][r] - delta);
                        }
                        ds[8 * kb + i] = N::pack2(v[0], v[1]);
                    }
#pragma unroll
                for (int n = 0; n < 4 * DB; ++n) {                // dQ^T += K^T dS^T
                    const int t2 = n / DB, db = n % DB;
                    const u32x4 b = {ds[4 * t2], ds[4 * t2 + 1], ds[4 * t2 + 2], ds[4 * t2 + 3]};
                    dq[db] = N::mfma(rd.transposed(k_tr, n), b, dq[db]);
                }
            }
            phase_barrier();                                    // everyone is done with this stage
        }
    }
    uint16_t *dQh = a.dQ + head_off;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 w;
            w[0] = N::pack2(dq[db][4 * g] * a.scale, dq[db][4 * g + 1] * a.scale);
            w[1] = N::pack2(dq[db][4 * g + 2] * a.scale, dq[db][4 * g + 3] * a.scale);
            *reinterpret_cast<u32x2 *>(dQh + (size_t)my_q * D + 32 * db + 8 * g + 4 * half) = w;
        }
}

// ---------------------------------------------------------------------------------------------------------
// dK, dV: a workgroup owns 128 keys (lane = key), walks the query tiles that see them.
// LDS stage: Q row-wise, Q transposed-pattern, dO row-wise, dO transposed-pattern, 64 logsumexps, 64 deltas.
// ---------------------------------------------------------------------------------------------------------
template <bool BF16, int D, bool MASKED>
__global__ void __launch_bounds__(kBwdWaves * 64, 1) fa_bwd_dkdv(const FaBwdArgs a)
{
    typedef Num<BF16> N;
    typedef TileReader<D> Reader;
    typedef TileLoader<D> Loader;
    constexpr int KS = Reader::KS, DB = Reader::DB, TILEB = Loader::TILEB, STAGEB = 4 * TILEB + 512, IPW = Loader::IPW;
    extern __shared__ __attribute__((aligned(1024))) char smem[];
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char *)smem;
    const int tid = threadIdx.x, lane = tid & 63, half = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int S = a.S;
    const int n_kblocks = S / 128;
    // one head per XCD at a time; key block 0 is seen by the most queries and goes first
    int bh, kblock;
    fa_item_decode((long long)blockIdx.x, a.BH, n_kblocks, 0, &bh, &kblock);
    const size_t head_off = (size_t)bh * S * D;
    const uint16_t *Qh = a.Q + head_off, *Kh = a.K + head_off, *Vh = a.V + head_off, *dOh = a.dO + head_off;
    const float *lse_h = a.lse + (size_t)bh * S, *delta_h = a.delta + (size_t)bh * S;
    const int k0 = kblock * 128, kw = k0 + wave * 32, my_k = kw + l32;

    u32x4 kf[KS], vf[KS];           // K^T and V^T as B operands: lane = (key, head-dim slice)
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        kf[s] = *reinterpret_cast<const u32x4 *>(Kh + (size_t)my_k * D + 16 * s + 8 * half);
        vf[s] = *reinterpret_cast<const u32x4 *>(Vh + (size_t)my_k * D + 16 * s + 8 * half);
    }
    const float c = a.scale * kLog2e;

    // the query tiles that see these keys: query i sees key j iff j - R <= i <= j + L (the forward bounds with
    // the two sides exchanged)
    int t0, t1, my_lo, my_hi;
    fa_tile_range(S, 64, a.R, a.L, k0, 128, &t0, &t1);
    fa_tile_range(S, 64, a.R, a.L, kw, 32, &my_lo, &my_hi);

    Reader rd; rd.init(lane);
    Loader ld; ld.init(wave, lane);
    auto issue = [&](int tile, int stage) __attribute__((always_inline)) {
        const uint32_t base = lds0 + stage * STAGEB;
        ld.load(Qh + (size_t)tile * 64 * D, base, true);
        ld.load(Qh + (size_t)tile * 64 * D, base + TILEB, false);
        ld.load(dOh + (size_t)tile * 64 * D, base + 2 * TILEB, true);
        ld.load(dOh + (size_t)tile * 64 * D, base + 3 * TILEB, false);
        if (wave == 0) dma_4(lse_h + tile * 64, lane, base + 4 * TILEB);
        if (wave == 1) dma_4(delta_h + tile * 64, lane, base + 4 * TILEB + 256);
    };
    // loads in flight per wave after one issue(): waves 0 and 1 have one more than the others
    f32x16 dk[DB], dv[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) { dk[db][r] = 0.0f; dv[db][r] = 0.0f; }

    if (t0 <= t1) {
        // from the last query tile down to the diagonal: every workgroup of a head then starts on the same tile
        // and the ones that run together keep reading the same tiles out of L2
        issue(t1, 0);
        wait_vm<0>();
#pragma unroll
        for (int s = 0; s < KS; ++s) asm volatile("" : "+v"(kf[s]), "+v"(vf[s]));
        for (int t = t1; t >= t0; --t) {
            const int stage = (t1 - t) & 1;
            if (t - 1 >= t0) {
                issue(t - 1, stage ^ 1);
                if (wave < 2) wait_vm<4 * IPW + 1>(); else wait_vm<4 * IPW>();
            } else wait_vm<0>();
            phase_barrier();
            if (my_lo <= t && t <= my_hi) {
                const uint32_t q_rows = lds0 + stage * STAGEB, q_tr = q_rows + TILEB, g_rows = q_rows + 2 * TILEB, g_tr = q_rows + 3 * TILEB;
                const uint32_t lse_s = q_rows + 4 * TILEB, delta_s = lse_s + 256;
                f32x16 sx[2], dp[2];     // [query block 0 / 1 of the tile]: rows = queries, column (lane) = key
#pragma unroll
                for (int r = 0; r < 16; ++r) { sx[0][r] = 0.0f; sx[1][r] = 0.0f; dp[0][r] = 0.0f; dp[1][r] = 0.0f; }
#pragma unroll
                for (int n = 0; n < 2 * KS; ++n) sx[n & 1] = N::mfma(rd.rows(q_rows, n), kf[n >> 1], sx[n & 1]);     // S = Q K^T
                // the logsumexp and delta of the accumulator rows: row r of block qb is query 32*qb + 8*(r/4) + 4*half + r%4
                const bool edge = MASKED && fa_tile_class(64, a.R, a.L, kw, 32, t) == 1;
                uint32_t pp[16];
#pragma unroll
                for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const u32x4 lraw = lds_read_b128(lse_s + (uint32_t)(32 * qb + 8 * g + 4 * half) * 4u);
                        float p[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            const int r = 4 * g + e;
                            const int i = t * 64 + 32 * qb + 8 * g + 4 * half + e;
                            p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sx[qb][r], c, -as_f32(lraw[e]) * kLog2e));
                            if (edge && (my_k > i + a.R || my_k < i - a.L)) p[e] = 0.0f;
                            sx[qb][r] = p[e];                    // keep P in fp32 for dS
                        }
                        pp[8 * qb + 2 * g] = N::pack2(p[0], p[1]);
                        pp[8 * qb + 2 * g + 1] = N::pack2(p[2], p[3]);
                    }
#pragma unroll
                for (int n = 0; n < 4 * DB; ++n) {                // dV^T += dO^T P
                    const int t2 = n / DB, db = n % DB;
                    const u32x4 b = {pp[4 * t2], pp[4 * t2 + 1], pp[4 * t2 + 2], pp[4 * t2 + 3]};
                    dv[db] = N::mfma(rd.transposed(g_tr, n), b, dv[db]);
                }
#pragma unroll
                for (int n = 0; n < 2 * KS; ++n) dp[n & 1] = N::mfma(rd.rows(g_rows, n), vf[n >> 1], dp[n & 1]);     // dP = dO V^T
#pragma unroll
                for (int qb = 0; qb < 2; ++qb)
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        const u32x4 draw = lds_read_b128(delta_s + (uint32_t)(32 * qb + 8 * g + 4 * half) * 4u);
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = sx[qb][4 * g + e] * (dp[qb][4 * g + e] - as_f32(draw[e]));
                        pp[8 * qb + 2 * g] = N::pack2(v[0], v[1]);     // now dS, same operand order
                        pp[8 * qb + 2 * g + 1] = N::pack2(v[2], v[3]);
                    }
#pragma unroll
                for (int n = 0; n < 4 * DB; ++n) {                // dK^T += Q^T dS
                    const int t2 = n / DB, db = n % DB;
                    const u32x4 b = {pp[4 * t2], pp[4 * t2 + 1], pp[4 * t2 + 2], pp[4 * t2 + 3]};
                    dk[db] = N::mfma(rd.transposed(q_tr, n), b, dk[db]);
                }
            }
            phase_barrier();
        }
    }
    uint16_t *dKh = a.dK + head_off, *dVh = a.dV + head_off;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            u32x2 wk, wv;
            wk[0] = N::pack2(dk[db][4 * g] * a.scale, dk[db][4 * g + 1] * a.scale);
            wk[1] = N::pack2(dk[db][4 * g + 2] * a.scale, dk[db][4 * g + 3] * a.scale);
            wv[0] = N::pack2(dv[db][4 * g], dv[db][4 * g + 1]);
            wv[1] = N::pack2(dv[db][4 * g + 2], dv[db][4 * g + 3]);
            *reinterpret_cast<u32x2 *>(dKh + (size_t)my_k * D + 32 * db + 8 * g + 4 * half) = wk;
            *reinterpret_cast<u32x2 *>(dVh + (size_t)my_k * D + 32 * db + 8 * g + 4 * half) = wv;
        }
}

template <bool BF16, int D, bool MASKED>
hipError_t launch_bwd(const FaBwdArgs &a, hipStream_t stream)
{
    constexpr int TILEB = 64 * D * 2;
    const long long rows = (long long)a.BH * a.S;
    hipLaunchKernelGGL((fa_bwd_delta<BF16, D>), dim3((unsigned)((rows + 255) / 256)), dim3(256), 0, stream, a);
    const unsigned grid = (unsigned)((long long)a.BH * (a.S / 128));
    const int smem_dq = 2 * 3 * TILEB, smem_dkdv = 2 * (4 * TILEB + 512);
    auto kq = fa_bwd_dq<BF16, D, MASKED>;
    auto kkv = fa_bwd_dkdv<BF16, D, MASKED>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kq), hipFuncAttributeMaxDynamicSharedMemorySize, smem_dq);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(kkv), hipFuncAttributeMaxDynamicSharedMemorySize, smem_dkdv);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(kq, dim3(grid), dim3(kBwdWaves * 64), smem_dq, stream, a);
    hipLaunchKernelGGL(kkv, dim3(grid), dim3(kBwdWaves * 64), smem_dkdv, stream, a);
    return hipGetLastError();
}

}  // namespace

hipError_t fa_launch_backward(const FaBwdArgs &a, int bf16, int D, int masked, hipStream_t stream)
{
#define FA_BWD_CASE(BF, DD, MK) \
    if (bf16 == BF && D == DD && masked == MK) return launch_bwd<BF != 0, DD, MK != 0>(a, stream);
    FA_BWD_CASE(0, 64, 0) FA_BWD_CASE(0, 64, 1) FA_BWD_CASE(0, 128, 0) FA_BWD_CASE(0, 128, 1)
    FA_BWD_CASE(1, 64, 0) FA_BWD_CASE(1, 64, 1) FA_BWD_CASE(1, 128, 0) FA_BWD_CASE(1, 128, 1)
#undef FA_BWD_CASE
    return hipErrorInvalidValue;
}
