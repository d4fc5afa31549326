// C ABI of the gfx950 FlashAttention forward library (see include/fa_fwd.h).
//
// Role of the reference's launcher run_flash_attention / run_kernel<>
// (reference src/flash_forward.h:369-665): argument checking, derived
// parameters, kernel selection and launch.  Unlike the reference it never
// exits, aborts or throws, launches asynchronously on the caller's stream,
// keeps no global descriptor state, and does not time or print.
#include <hip/hip_runtime.h>
#include <dlfcn.h>
#include <math.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "fa_fwd.h"
#include "fa_bwd.h"
#include "fa_bwd_args.h"
#include "fa_bwd_layout.h"
#include "fa_device_state.h"
#include "fa_kernel_args.h"
#include "fa_sched.h"

hipError_t fa_launch_forward_contiguous(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                        hipStream_t stream);
hipError_t fa_launch_forward_strided(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                     hipStream_t stream);
hipError_t fa_launch_forward_general(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                     hipStream_t stream);
hipError_t fa_launch_forward_dropout(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                     hipStream_t stream);
hipError_t fa_launch_forward_dropout_regular(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                             hipStream_t stream);
hipError_t fa_launch_combine_splits(const FaKernelArgs &a, int bf16, int D, hipStream_t stream);
hipError_t fa_launch_backward(const FaBwdArgs &a, int bf16, int D, int masked, int general, int alibi, int compute_units,
                              hipStream_t stream, bool configure_only = false);
hipError_t fa_launch_backward_dropout(const FaBwdArgs &a, int bf16, int D, int alibi, int compute_units, hipStream_t stream,
                                      bool configure_only = false);
hipError_t fa_launch_backward_strided(const FaBwdArgs &a, int bf16, int D, int masked, int compute_units, hipStream_t stream,
                                      bool configure_only = false);
// the LDS opt-in (hipFuncSetAttribute) of every kernel instantiation of a translation unit, for the current device
hipError_t fa_configure_forward_contiguous();
hipError_t fa_configure_forward_strided();
hipError_t fa_configure_forward_general();
hipError_t fa_configure_forward_dropout();
hipError_t fa_configure_forward_dropout_regular();
hipError_t fa_configure_backward();
hipError_t fa_configure_backward_dropout();
hipError_t fa_launch_backward_dropout_regular(const FaBwdArgs &a, int bf16, int D, int masked, int strided, int compute_units,
                                              hipStream_t stream, bool configure_only = false);
hipError_t fa_configure_backward_dropout_regular();
hipError_t fa_launch_backward_alibi_regular(const FaBwdArgs &a, int bf16, int D, int masked, int strided, int compute_units,
                                            hipStream_t stream, bool configure_only = false);
hipError_t fa_configure_backward_alibi_regular();
hipError_t fa_configure_backward_strided();

namespace {
constexpr int kBlockKeysHost = 64;
constexpr int kComputeUnits = 256;      // MI355X; the persistent grid is sized from the device at run time

// Workgroup shape for a problem.  The 8-wave kernel (256 query rows, one workgroup per CU) shares every K/V
// tile among more rows; the 4-wave kernel (128 rows, two workgroups per CU, each with its own barrier, so that the
// two waves of a SIMD are never lined up by one) has twice as many, smaller work items.  It wins when there are
// too few of the large items to fill and balance the chip, and when the items are short, i.e. when no query sees
// more than 1024 keys (at head dimension 64, where a tile carries half the matrix work per barrier, 4096 under a
// mask and 2048 without one): short sequences, and windows on long ones.  Measured, causal fp16, 4 waves against 8, TFLOP/s in one process: B8 H32
// S1024 D64 504 against 432, B8 H16 S1024 D64 443 against 391, B16 H16 S512 D64 275 against 252, B8 H32 S1024 D128 653
// against 590, B16 H16 S512 D128 369 against 340, c2 (B4 H16 S2048 D64) 568-580 against 541-563, B4 H32 S2048 D64 638
// against 626; windows: 512 keys at B1 H32 S16384 D128 604 against 546, 1024 keys at B2 H32 S8192 D64 618 against 578,
// 256 keys at B4 H32 S2048 D64 275 against 241; without a mask B8 H32 S1024 D64 734 against 718; and the other way
// round a window of 2048 keys at B1 H32 S16384 D128 867 against 899, B2 H32 S4096 D128 907 against 958, B1 H32 S8192
// D64 796 against 818, c3 973-1002 against 1029-1051; level: c4 (window 1024, D128, which stays with 8 waves) 780
// against 782.  Head dimension 64 at 4096 keys: causal B2 H32 751 against 744, B8 H32 774 against 748, B1 H16 455
// against 443, windows of 3000 and 4096 keys at B2 H32 S8192 728 against 688 and 736 against 683; without a mask B2 H32
// S4096 868 against 888.
// (`keys`: the largest number of keys a query can see, the key length without a mask)
int waves_for(int B, int N, int S, int d, long long keys, bool masked)
{
    if (S < 256) return 4;              // (few queries per head, e.g. decoding: a 256-row block would be mostly empty)
    if (keys <= (d == 64 ? (masked ? 4096 : 2048) : 1024)) return 4;
    const long long big_items = (long long)B * N * ((S + 255) / 256);
    return big_items >= 2LL * kComputeUnits ? 8 : 4;
}
// the same from the mask as the boundary states it
int waves_for_mask(int B, int N, int S, int S_kv, int d, int is_causal, int window_left, int window_right)
{
    const int sk = S_kv > 0 ? S_kv : S, s_max = sk > S ? sk : S;
    int L, R;
    fa_mask_bounds(s_max, is_causal, window_left, window_right, &L, &R);
    const long long keys = (long long)L + R + 1;
    return waves_for(B, N, S, d, keys < sk ? keys : sk, L < s_max || R < s_max);
}
int waves_of(const fa_fwd_params *p)
{
    return waves_for_mask(p->B, p->N, p->S, p->S_kv, p->d, p->is_causal, p->window_size_left, p->window_size_right);
}

thread_local char g_last_error[256] = "";

std::atomic<unsigned> g_capture_ticket[kFaMaxDevices];     // captured queue launches so far, per device
// Eager launches: which stream owns which counter set of a device.  A stream is named by its handle AND the id
// the runtime gave it at creation (hipStreamGetId): a handle value can come back for a new stream after the old
// one was destroyed, while the old stream's last launch may still be running on its counters; the id never does.
struct SlotOwner {
    uintptr_t handle;           // 0 = free
    unsigned long long id;
};
std::mutex g_slot_mutex;
// hipStreamGetId exists from HIP 7.1 on; a process may have loaded an older runtime (PyTorch wheels bring their
// own), so it is looked up at run time.  Without it a stream is named by its handle alone, and a caller that
// destroys streams has to release their sets first (fa_release_work_queue).
typedef hipError_t (*StreamIdFn)(hipStream_t, unsigned long long *);
bool stream_id(hipStream_t stream, unsigned long long *id)
{
    static const StreamIdFn fn = reinterpret_cast<StreamIdFn>(dlsym(RTLD_DEFAULT, "hipStreamGetId"));
    *id = 0;
    return fn == nullptr || fn(stream, id) == hipSuccess;
}
SlotOwner g_slot_owner[kFaMaxDevices][kFaEagerQueueSlots];

// A counter set for one FA_SCHED_QUEUE launch, or null when none can be given safely (the caller then walks the
// list with the fixed snake: same results, no counters).  Eager launches: a set belongs to a stream -- launches on
// one stream run one after the other, so they may share it, and every launch leaves it rewound; a device hands out
// sixteen sets, to the first sixteen streams that ask, and a stream keeps its set until fa_release_work_queue or
// fa_reset_work_queues; further streams get none.  hipStreamPerThread gets none either: it is one handle value
// for a different stream in every host thread.  A launch that is being captured into a graph keeps its set for
// every replay of that graph, and a replay may run next to anything: every captured launch gets a set of its own
// from the remaining 240, for good, and when those are used up captured launches get none.  No two launches that
// can run at the same time ever share counters.
unsigned *work_queue_for_launch(const FaDeviceState *ds, hipStream_t stream)
{
    if (stream == hipStreamPerThread) return nullptr;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    const bool capturing = stream != nullptr && stream != hipStreamLegacy && hipStreamIsCapturing(stream, &status) == hipSuccess &&
                           status == hipStreamCaptureStatusActive;
    if (capturing) {
        const unsigned n = g_capture_ticket[fa_launch_device()].fetch_add(1u, std::memory_order_relaxed);
        if (n >= (unsigned)(kFaQueueSlots - kFaEagerQueueSlots)) return nullptr;
        return ds->queues + 16u * ((unsigned)kFaEagerQueueSlots + n);
    }
    // (the two names of the legacy default stream are one stream)
    const bool legacy = stream == nullptr || stream == hipStreamLegacy;
    const uintptr_t handle = legacy ? (uintptr_t)1 : reinterpret_cast<uintptr_t>(stream);
    unsigned long long id = 0;
    if (!legacy && !stream_id(stream, &id)) return nullptr;
    std::lock_guard<std::mutex> lock(g_slot_mutex);
    SlotOwner *owners = g_slot_owner[fa_launch_device()];
    int free_slot = -1;
    for (int i = 0; i < kFaEagerQueueSlots; ++i) {
        if (owners[i].handle == handle && owners[i].id == id) return ds->queues + 16u * (unsigned)i;
        if (owners[i].handle == 0 && free_slot < 0) free_slot = i;
    }
    if (free_slot < 0) return nullptr;
    owners[free_slot] = SlotOwner{handle, id};
    return ds->queues + 16u * (unsigned)free_slot;
}

int device_fail(hipError_t e, const char *what)
{
    snprintf(g_last_error, sizeof(g_last_error), "%s: %s", what, hipGetErrorString(e));
    return FA_ERR_DEVICE;
}
}  // namespace

extern "C" {

const char *fa_strerror(int status)
{
    switch (status) {
    case FA_OK: return "ok";
    case FA_ERR_NULL_POINTER: return "Q, K, V or O is NULL";
    case FA_ERR_BAD_SHAPE: return "batch, heads and seqlen must be positive";
    case FA_ERR_HEAD_DIM: return "head_dim must be 64 or 128";
    case FA_ERR_SEQLEN_MULTIPLE: return "reserved (seqlen no longer has to be a multiple of 128)";
    case FA_ERR_WORKSPACE: return "needs a 16-byte aligned workspace of fa_fwd_workspace_bytes() (split_num > 1) or fa_bwd_workspace_bytes() bytes";
    case FA_ERR_LAYOUT: return "strides must be multiples of 8 elements (row strides at least head_dim), n_kv_heads must divide heads, pointers must be 16-byte aligned";
    case FA_ERR_UNSUPPORTED: return "dropout_prob must be at least 0 and below 1";
    case FA_ERR_DTYPE: return "dtype must be FA_DTYPE_F16 or FA_DTYPE_BF16";
    case FA_ERR_SCALE: return "softmax_scale must be finite and positive";
    case FA_ERR_DEVICE: return "HIP runtime error";
    case FA_ERR_NO_DEVICE: return "no gfx950 device visible";
    case FA_ERR_TOO_LARGE: return "problem too large for the kernel's index range";
    case FA_ERR_SCRATCH_LIMIT: return "the partial results of this call exceed the library's static scratch (fa_fwd_static_scratch_bytes): use fewer splits or fa_fwd with a workspace";
    default: return "unknown status";
    }
}

const char *fa_last_device_error(void) { return g_last_error; }

int fa_sched_block_rows(int B, int N, int S, int d, int is_causal, int window_left, int window_right)
{
    return 32 * waves_for_mask(B, N, S, S, d, is_causal, window_left, window_right);
}
int fa_sched_block_keys(int d) { (void)d; return kBlockKeysHost; }

long long fa_sched_num_items(int B, int N, int S, int d, int is_causal, int window_left, int window_right)
{
    const int br = fa_sched_block_rows(B, N, S, d, is_causal, window_left, window_right);
    return (long long)B * N * ((S + br - 1) / br);
}

int fa_sched_item(int B, int N, int S, int d, int is_causal, int window_left, int window_right,
                  long long item, int *bh, int *q_begin)
{
    if (B <= 0 || N <= 0 || S <= 0 || !bh || !q_begin) return FA_ERR_BAD_SHAPE;
    const int br = fa_sched_block_rows(B, N, S, d, is_causal, window_left, window_right);
    const int nqb = (S + br - 1) / br;
    if (item < 0 || item >= (long long)B * N * nqb) return FA_ERR_BAD_SHAPE;
    int L, R, qb;
    fa_mask_bounds(S, is_causal, window_left, window_right, &L, &R);
    fa_item_decode(item, B * N, nqb, (L < S || R < S) ? 1 : 0, bh, &qb);
    *q_begin = qb * br;
    return FA_OK;
}

int fa_sched_heads(int N, int n_kv_heads, int bh, int *batch, int *q_head, int *kv_head)
{
    const int hk = n_kv_heads > 0 ? n_kv_heads : N;
    if (N <= 0 || hk > N || N % hk != 0 || bh < 0 || !batch || !q_head || !kv_head) return FA_ERR_BAD_SHAPE;
    *batch = fa_strided_heads(bh, N, hk, q_head, kv_head);
    return FA_OK;
}

void fa_sched_tile_range(int S, int block_keys, int is_causal, int window_left, int window_right,
                         int q_begin, int rows, int *tile_lo, int *tile_hi)
{
    int L, R;
    fa_mask_bounds(S, is_causal, window_left, window_right, &L, &R);
    fa_tile_range(S, block_keys, L, R, q_begin, rows, tile_lo, tile_hi);
}

int fa_sched_classify(int block_keys, int is_causal, int window_left, int window_right,
                      int q_begin, int rows, int tile)
{
    // "unbounded" only has to exceed every reachable |i-j|
    const int big = 0x3fffffff;
    int L = window_left < 0 ? big : window_left;
    int R = window_right < 0 ? big : window_right;
    if (is_causal) R = 0;
    return fa_tile_class(block_keys, L, R, q_begin, rows, tile);
}

long long fa_count_pairs(int S, int is_causal, int window_left, int window_right)
{
    int L, R;
    fa_mask_bounds(S, is_causal, window_left, window_right, &L, &R);
    long long pairs = 0;
    for (int i = 0; i < S; ++i) {
        int lo = i - L < 0 ? 0 : i - L;
        int hi = i + R > S - 1 ? S - 1 : i + R;
        pairs += hi - lo + 1;
    }
    return pairs;
}

double fa_algorithmic_flops(int B, int N, int S, int d, int is_causal, int window_left, int window_right)
{
    return 4.0 * (double)B * (double)N * (double)d * (double)fa_count_pairs(S, is_causal, window_left, window_right);
}

int fa_dropout_threshold(float dropout_prob)
{
    if (!(dropout_prob > 0.0f)) return 0;
    const long t = lrintf(dropout_prob * 256.0f);
    return t > 255 ? 255 : (int)t;
}

int fa_dropout_keep(unsigned long long seed, long long bh, int i, int j, int threshold)
{
    // One Philox4x32-10 block per (query, 32-key block, (j / 4) % 2): sixteen bytes for sixteen keys.
    uint32_t c0 = (uint32_t)(2 * (j >> 5) + ((j >> 2) & 1)), c1 = (uint32_t)i, c2 = (uint32_t)bh, c3 = 0x44524F50u;
    uint32_t k0 = (uint32_t)(seed & 0xffffffffull), k1 = (uint32_t)(seed >> 32);
    for (int round = 0; round < 10; ++round) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        c1 = (uint32_t)p1; c3 = (uint32_t)p0; c0 = n0; c2 = n2;
        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
    }
    const uint32_t w[4] = {c0, c1, c2, c3};
    const int r = 4 * ((j & 31) >> 3) + (j & 3);
    return (int)((w[r >> 2] >> (8 * (r & 3))) & 255u) >= threshold;
}

namespace {
int key_tiles(const fa_fwd_params *p) { return ((p->S_kv > 0 ? p->S_kv : p->S) + kBlockKeysHost - 1) / kBlockKeysHost; }
// splits actually used: at most one per key tile
// Query heads per K/V head packed into the rows of one work item (1 = not packed): when there are few
// queries behind long keys (decoding), all query heads of a K/V head fit one 128-row workgroup and K and V
// are then read once per group instead of once per query head.
int packed_group(const fa_fwd_params *p)
{
    const int hk = p->n_kv_heads > 0 ? p->n_kv_heads : p->N;
    if (hk <= 0 || hk >= p->N || p->N % hk != 0) return 1;
    const int group = p->N / hk, sk = p->S_kv > 0 ? p->S_kv : p->S;
    if (sk <= p->S) return 1;                                  // queries must sit behind earlier keys
    if ((long long)group * p->S > 32LL * waves_of(p)) return 1;
    return group;
}
// work items before key splits
long long base_items(const fa_fwd_params *p)
{
    const int pack = packed_group(p);
    if (pack > 1) return (long long)p->B * (p->N / pack);
    return fa_sched_num_items(p->B, p->N, p->S, p->d, p->is_causal, p->window_size_left, p->window_size_right);
}
int effective_splits(const fa_fwd_params *p)
{
    if (p->split_num <= 1) return 1;
    const int tiles = key_tiles(p);
    return p->split_num < tiles ? p->split_num : tiles;
}
}  // namespace

unsigned long long fa_fwd_workspace_bytes(const fa_fwd_params *p)
{
    if (!p || p->B <= 0 || p->N <= 0 || p->S <= 0 || p->d <= 0) return 0;
    const int n = effective_splits(p);
    if (n <= 1) return 0;
    return (unsigned long long)n * p->B * p->N * p->S * (unsigned long long)(p->d + 1) * 4ull;
}

int fa_fwd_suggest_splits(const fa_fwd_params *p)
{
    if (!p || p->B <= 0 || p->N <= 0 || p->S <= 0) return 1;
    // work items without splits against the workgroups the device keeps resident; split until the device is
    // filled once (the items of such a problem are all alike, so one full round has no tail; measured against
    // filling it twice: 98 against 106 us on B16 H32/8 S1 S_kv8192, 53 against 61 us on B8 H32/8 S4 S_kv8192,
    // 370 against 361 us on B4 H32 S1 S_kv32768), with at least four key tiles (256 keys) per split
    const long long items = base_items(p);
    const long long resident = (long long)kComputeUnits * (waves_of(p) == 8 ? 1 : 2);
    if (items >= resident) return 1;
    long long n = (resident + items - 1) / items;
    const long long cap = key_tiles(p) / 4;
    if (n > cap) n = cap;
    return n < 1 ? 1 : (int)n;
}

namespace {
int validate_layout(const fa_fwd_params *p);
// everything but the workspace of a call with key splits
int validate_no_workspace(const fa_fwd_params *p)
{
    if (!p || !p->Q || !p->K || !p->V || !p->O) return FA_ERR_NULL_POINTER;
    if (p->B <= 0 || p->N <= 0 || p->S <= 0) return FA_ERR_BAD_SHAPE;
    if (p->d != 64 && p->d != 128) return FA_ERR_HEAD_DIM;
    if (p->dtype != FA_DTYPE_F16 && p->dtype != FA_DTYPE_BF16) return FA_ERR_DTYPE;
    if (!(p->dropout_prob >= 0.0f) || !(p->dropout_prob < 1.0f)) return FA_ERR_UNSUPPORTED;
    if (!(p->softmax_scale > 0.0f) || !isfinite(p->softmax_scale)) return FA_ERR_SCALE;
    const long long bh = (long long)p->B * p->N;
    if (bh > 0x7fffffffLL || fa_sched_num_items(p->B, p->N, p->S, p->d, p->is_causal, p->window_size_left, p->window_size_right) > 0x7fffffffLL) return FA_ERR_TOO_LARGE;
    if (p->S_kv < 0) return FA_ERR_BAD_SHAPE;
    if ((long long)p->S + (p->S_kv > 0 ? p->S_kv : p->S) > 0x3fffffffLL) return FA_ERR_TOO_LARGE;   // tile and mask arithmetic is 32-bit
    if (base_items(p) * effective_splits(p) > 0x7fffffffLL) return FA_ERR_TOO_LARGE;
    return validate_layout(p);
}
}  // namespace

int fa_fwd_validate(const fa_fwd_params *p)
{
    const int st = validate_no_workspace(p);
    if (st != FA_OK) return st;
    if (effective_splits(p) > 1 && (p->workspace == nullptr || reinterpret_cast<uintptr_t>(p->workspace) % 16 != 0 ||
                                    p->workspace_bytes < fa_fwd_workspace_bytes(p))) return FA_ERR_WORKSPACE;
    return FA_OK;
}

namespace {
int validate_layout(const fa_fwd_params *p)
{
    if (p->n_kv_heads < 0 || (p->n_kv_heads > 0 && p->N % p->n_kv_heads != 0)) return FA_ERR_LAYOUT;
    const void *ptrs[4] = {p->Q, p->K, p->V, p->O};
    const long long *strides[4] = {p->q_strides, p->k_strides, p->v_strides, p->o_strides};
    for (int t = 0; t < 4; ++t) {
        if (reinterpret_cast<uintptr_t>(ptrs[t]) % 16 != 0) return FA_ERR_LAYOUT;
        const long long *st = strides[t];
        if (st[0] == 0 && st[1] == 0 && st[2] == 0) continue;       // contiguous
        for (int k = 0; k < 3; ++k)
            if (st[k] < 0 || st[k] % 8 != 0) return FA_ERR_LAYOUT;
        if (st[2] < p->d) return FA_ERR_LAYOUT;
        if (st[2] > (1LL << 24)) return FA_ERR_TOO_LARGE;           // per-lane byte offsets inside a tile are 32-bit
        // an output whose batch or head stride is zero would have several writers per element
        if (t == 3 && ((p->B > 1 && st[0] == 0) || (p->N > 1 && st[1] == 0))) return FA_ERR_LAYOUT;
    }
    return FA_OK;
}

// The forward pass with the partial results of key splits in `workspace` (ignored without splits).
int forward(const fa_fwd_params *p, void *workspace, const FaDeviceState *ds, void *stream)
{
    FaKernelArgs a;
    a.Q = static_cast<const uint16_t *>(p->Q);
    a.K = static_cast<const uint16_t *>(p->K);
    a.V = static_cast<const uint16_t *>(p->V);
    a.O = static_cast<uint16_t *>(p->O);
    a.lse = p->L;
    a.alibi = p->alibi_slopes_ptr;
    a.H = p->N;
    a.BH = p->B * p->N;
    a.S = p->S;
    // layout: contiguous [B,N,S,d] unless strides are given; K and V have n_kv_heads heads
    a.Hk = p->n_kv_heads > 0 ? p->n_kv_heads : p->N;
    a.Sk = p->S_kv > 0 ? p->S_kv : p->S;
    a.n_splits = effective_splits(p);
    a.tiles_per_split = (key_tiles(p) + a.n_splits - 1) / a.n_splits;
    a.o_part = static_cast<float *>(workspace);
    a.lse_part = a.o_part != nullptr ? a.o_part + (size_t)a.n_splits * p->B * p->N * p->S * p->d : nullptr;
    a.pack = packed_group(p);
    bool general = a.pack > 1 || p->S % 128 != 0 || a.Sk != p->S || a.n_splits > 1;
    // the regular problem, not stored contiguous [B,N,S,d], or with K/V heads shared by groups of query heads
    bool strided = a.Hk != p->N;
    {
        const long long *strides[4] = {p->q_strides, p->k_strides, p->v_strides, p->o_strides};
        long long eff[4][3];
        for (int t = 0; t < 4; ++t) {
            const long long heads = (t == 1 || t == 2) ? a.Hk : p->N;
            const long long len = (t == 1 || t == 2) ? a.Sk : p->S;
            const long long dense[3] = {heads * len * p->d, len * p->d, p->d};
            const long long *st = strides[t];
            const bool given = st[0] != 0 || st[1] != 0 || st[2] != 0;
            for (int k = 0; k < 3; ++k) {
                eff[t][k] = given ? st[k] : dense[k];
                if (eff[t][k] != dense[k]) strided = true;
            }
        }
        a.q_bs = eff[0][0]; a.q_hs = eff[0][1]; a.q_rs = (int)eff[0][2];
        a.k_bs = eff[1][0]; a.k_hs = eff[1][1]; a.k_rs = (int)eff[1][2];
        a.v_bs = eff[2][0]; a.v_hs = eff[2][1]; a.v_rs = (int)eff[2][2];
        a.o_bs = eff[3][0]; a.o_hs = eff[3][1]; a.o_rs = (int)eff[3][2];
    }
    const int waves = waves_of(p);
    const int block_rows = 32 * waves;
    a.n_qblocks = a.pack > 1 ? 1 : (p->S + block_rows - 1) / block_rows;
    const int s_max = a.Sk > p->S ? a.Sk : p->S;        // stands in for "unbounded"
    fa_mask_bounds(s_max, p->is_causal, p->window_size_left, p->window_size_right, &a.L, &a.R);
    // (a sequence that ends inside a 64-key tile needs the element mask on that tile, whatever the mask)
    const int masked = (a.L < s_max || a.R < s_max || a.Sk % kBlockKeysHost != 0) ? 1 : 0;
    a.descending = (a.L < s_max || a.R < s_max) ? 1 : 0;
    a.scale = p->softmax_scale;
    a.scale_log2e = p->softmax_scale * 1.44269504088896340736f;
    a.n_items = (long long)(a.BH / a.pack) * a.n_qblocks * a.n_splits;

    // Dispatch mode launches one workgroup per item, in list order; the hardware hands them to CUs as these
    // free up, which is a longest-first greedy schedule.  Persistent mode launches one resident set of
    // workgroups that walk the list themselves.
    long long grid = a.n_items;
    a.queue = nullptr;
    const long long resident = (long long)ds->compute_units * (waves == 8 ? 1 : 2);
    // FA_SCHED_AUTO: with at most one item per resident workgroup there is nothing to schedule (and the
    // queue's counter round trips, 2.3 us each, would double the run time of a 7 us problem).  With fewer than
    // eight items per workgroup the fixed snake wins: it pairs every long item with a short one, knows its next
    // item without asking, and its items' loads can be requested before the current item's epilogue without a
    // counter in between -- causal fp16 problems, snake against queue: B8 H32 S1024 D64 (four items per workgroup)
    // 67 against 100 us, B4 H32 S2048 D64 (four) 111 against 138, B2 H32 S4096 D128 (four) 290 against 312, c2 (two)
    // 611 against 448 TFLOP/s.  At eight per workgroup the two are level (c3 1016 against 1018 TFLOP/s, B1 H32 S16384
    // 2097 us both); beyond, the queue's balancing is worth more than its counters cost (c5, 32 items per workgroup:
    // 16.2 against 17.0 ms; B8 H32 S8192 D64 2.75 against 2.80 ms).
    int sched = p->sched;
    // Items that are all alike (no mask, or a window of at most half the length: all but the first few query blocks
    // of a head see the same number of tiles) need no balancing either, and the fixed order saves them the
    // counters' barriers: c4 766 against 748 TFLOP/s, c3's shape without a mask 1101 against 1096.
    if (sched == FA_SCHED_AUTO) {
        const bool alike = !a.descending || 2LL * a.L <= (long long)p->S;
        sched = a.n_items <= resident ? FA_SCHED_DISPATCH : (a.n_items < 8 * resident || alike) ? FA_SCHED_PERSISTENT : FA_SCHED_QUEUE;
    }
    if (sched == FA_SCHED_PERSISTENT || sched == FA_SCHED_QUEUE) {
        if (grid > resident) grid = resident;
        if (sched == FA_SCHED_QUEUE) a.queue = work_queue_for_launch(ds, static_cast<hipStream_t>(stream));
    }
    const int shape = waves == 8 ? 0 : 1;
    // dropout: p in units of 1/256 (a key is kept iff its random byte is >= the threshold)
    a.drop_threshold = (unsigned)fa_dropout_threshold(p->dropout_prob);
    a.drop_scale = 256.0f / (256.0f - (float)a.drop_threshold);
    a.seed_lo = (unsigned)(p->seed & 0xffffffffull);
    a.seed_hi = (unsigned)(p->seed >> 32);
    a.exact_first_rows = p->exact_first_rows != 0;
#ifdef FA_CHECK_RING
    a.ring_check = ds->ring_check;
#endif
    hipError_t e = (a.drop_threshold != 0 ? (general ? fa_launch_forward_dropout : fa_launch_forward_dropout_regular)
                    : general ? fa_launch_forward_general
                    : strided ? fa_launch_forward_strided : fa_launch_forward_contiguous)(
        a, p->dtype == FA_DTYPE_BF16, p->d, masked, shape, (unsigned)grid, static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return device_fail(e, "forward launch");
    if (a.n_splits > 1) {
        e = fa_launch_combine_splits(a, p->dtype == FA_DTYPE_BF16, p->d, static_cast<hipStream_t>(stream));
        if (e != hipSuccess) return device_fail(e, "combine launch");
    }
    return FA_OK;
}
}  // namespace

int fa_init(void)
{
    const FaDeviceState *ds = nullptr;
    hipError_t e = fa_device_state(&ds);
    if (e != hipSuccess) return device_fail(e, "device set-up");
    // everything a first launch would otherwise do besides the launch itself: after this call no entry point makes
    // a HIP call on this device that is not a stream operation (which is what a stream capture needs)
    hipError_t (*const configure[])() = {fa_configure_forward_contiguous, fa_configure_forward_strided, fa_configure_forward_general,
                                         fa_configure_forward_dropout, fa_configure_forward_dropout_regular, fa_configure_backward, fa_configure_backward_dropout,
                                         fa_configure_backward_strided, fa_configure_backward_dropout_regular, fa_configure_backward_alibi_regular};
    for (auto fn : configure) {
        e = fn();
        if (e != hipSuccess) return device_fail(e, "kernel set-up");
    }
    return FA_OK;
}

int fa_fwd(const fa_fwd_params *p, void *stream)
{
    const int st = fa_fwd_validate(p);
    if (st != FA_OK) return st;
    const FaDeviceState *ds = nullptr;
    const hipError_t e = fa_device_state(&ds);
    if (e != hipSuccess) return device_fail(e, "device set-up");
    return forward(p, p->workspace, ds, stream);
}

unsigned long long fa_fwd_static_scratch_bytes(void) { return kFaStaticScratchBytes; }

int fa_fwd_split_static(const fa_fwd_params *p, void *stream)
{
    const int st = validate_no_workspace(p);
    if (st != FA_OK) return st;
    if (fa_fwd_workspace_bytes(p) > kFaStaticScratchBytes) return FA_ERR_SCRATCH_LIMIT;
    const FaDeviceState *ds = nullptr;
    const hipError_t e = fa_device_state(&ds);      // first call on a device: looks the two arrays up, no allocation
    if (e != hipSuccess) return device_fail(e, "device set-up");
    // the kernels get the array's device address, exactly as they get a caller's workspace in fa_fwd
    return forward(p, ds->scratch, ds, stream);
}

#ifdef FA_CHECK_RING
// Checking build only (libfa_fwd_gfx950_check.so): waits for the device, returns how many 16-byte comparisons the
// forward kernels' ring checks have made and how many of them found other bytes in LDS than the tile the
// iteration expected, and sets both counters back to zero.
int fa_debug_ring_counts(unsigned long long *checks, unsigned long long *violations)
{
    const FaDeviceState *ds = nullptr;
    hipError_t e = fa_device_state(&ds);
    if (e != hipSuccess) return device_fail(e, "device set-up");
    unsigned long long host[2] = {0, 0};
    e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipMemcpy(host, ds->ring_check, sizeof(host), hipMemcpyDeviceToHost);
    if (e == hipSuccess) e = hipMemset(ds->ring_check, 0, sizeof(host));
    if (e != hipSuccess) return device_fail(e, "ring check counters");
    if (checks) *checks = host[0];
    if (violations) *violations = host[1];
    return FA_OK;
}
#endif

int fa_reset_work_queues(void)
{
    const FaDeviceState *ds = nullptr;
    hipError_t e = fa_device_state(&ds);
    if (e != hipSuccess) return device_fail(e, "device set-up");
    e = hipDeviceSynchronize();
    if (e != hipSuccess) return device_fail(e, "synchronize");
    e = hipMemset(ds->queues, 0, (size_t)kFaQueueSlots * 16 * sizeof(unsigned));
    if (e != hipSuccess) return device_fail(e, "work queue reset");
    // (nothing is in flight after the synchronisation: streams may claim their sets anew)
    std::lock_guard<std::mutex> lock(g_slot_mutex);
    for (int i = 0; i < kFaEagerQueueSlots; ++i) g_slot_owner[fa_launch_device()][i] = SlotOwner{0, 0};
    return FA_OK;
}

int fa_release_work_queue(void *stream_handle)
{
    hipStream_t stream = static_cast<hipStream_t>(stream_handle);
    const FaDeviceState *ds = nullptr;
    hipError_t e = fa_device_state(&ds);
    if (e != hipSuccess) return device_fail(e, "device set-up");
    if (stream == hipStreamPerThread) return FA_OK;             // never owns a set
    const bool legacy = stream == nullptr || stream == hipStreamLegacy;
    const uintptr_t handle = legacy ? (uintptr_t)1 : reinterpret_cast<uintptr_t>(stream);
    unsigned long long id = 0;
    if (!legacy && !stream_id(stream, &id)) return device_fail(hipErrorInvalidHandle, "hipStreamGetId");
    // the stream's last launch must have left the set rewound before another stream may take it
    e = hipStreamSynchronize(stream);
    if (e != hipSuccess) return device_fail(e, "synchronize");
    std::lock_guard<std::mutex> lock(g_slot_mutex);
    SlotOwner *owners = g_slot_owner[fa_launch_device()];
    for (int i = 0; i < kFaEagerQueueSlots; ++i)
        if (owners[i].handle == handle && owners[i].id == id) owners[i] = SlotOwner{0, 0};
    return FA_OK;
}

int run_flash_attention(int B, int N, int S, int d, void *Q, void *K, void *V, void *O, void *L, void *M,
                        int Is_dropout, int Is_causal, int Is_local, int Has_alibi, int window_size,
                        float *alibi_slopes, float dropout_prob, void *states)
{
    (void)M;
    (void)states;
    if (Has_alibi && alibi_slopes == nullptr) return FA_ERR_NULL_POINTER;
    if (d <= 0) return FA_ERR_HEAD_DIM;
    fa_fwd_params p;
    memset(&p, 0, sizeof(p));
    p.Q = Q; p.K = K; p.V = V; p.O = O;
    p.L = static_cast<float *>(L);
    p.B = B; p.N = N; p.S = S; p.d = d;
    p.softmax_scale = (float)(1.0 / sqrt((double)d));      // flash_forward.h:639
    p.dropout_prob = Is_dropout ? dropout_prob : 0.0f;
    p.seed = 48;                                             // the seed main() gives its curand states, main.cu:93
    p.alibi_slopes_ptr = Has_alibi ? alibi_slopes : nullptr;      // [N] device floats, main.cu:36-45
    p.window_size_left = Is_local ? window_size : -1;      // flash_forward.h:640-641, mask.h:55
    p.window_size_right = Is_local ? window_size : -1;
    if (Is_local && window_size < 0) { p.window_size_left = p.window_size_right = 0; }
    p.dtype = FA_DTYPE_F16;
    p.is_causal = Is_causal ? 1 : 0;
    const int st = fa_fwd(&p, nullptr);
    if (st != FA_OK) return st;
    hipError_t e = hipStreamSynchronize(nullptr);           // flash_forward.h:655
    if (e != hipSuccess) return device_fail(e, "synchronize");
    return FA_OK;
}

/* ---------------- thin device layer ---------------- */
int fa_dev_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return 0;
    return n;
}

int fa_dev_name(char *buf, size_t len, int *compute_units, int *clock_khz)
{
    hipDeviceProp_t prop;
    hipError_t e = hipGetDeviceProperties(&prop, 0);
    if (e != hipSuccess) return device_fail(e, "hipGetDeviceProperties");
    if (buf && len) { snprintf(buf, len, "%s (%s)", prop.name, prop.gcnArchName); }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (clock_khz) *clock_khz = prop.clockRate;
    return FA_OK;
}

#define FA_DEV(call, what) do { hipError_t e_ = (call); if (e_ != hipSuccess) return device_fail(e_, what); } while (0)

int fa_dev_malloc(void **ptr, size_t bytes) { if (!ptr) return FA_ERR_NULL_POINTER; FA_DEV(hipMalloc(ptr, bytes), "hipMalloc"); return FA_OK; }
int fa_dev_free(void *ptr) { FA_DEV(hipFree(ptr), "hipFree"); return FA_OK; }
int fa_dev_h2d(void *dst, const void *src, size_t bytes) { FA_DEV(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice), "hipMemcpy H2D"); return FA_OK; }
int fa_dev_d2h(void *dst, const void *src, size_t bytes) { FA_DEV(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost), "hipMemcpy D2H"); return FA_OK; }
int fa_dev_memset(void *dst, int value, size_t bytes) { FA_DEV(hipMemset(dst, value, bytes), "hipMemset"); return FA_OK; }
int fa_dev_sync(void) { FA_DEV(hipDeviceSynchronize(), "hipDeviceSynchronize"); return FA_OK; }
int fa_event_create(void **ev)
{
    if (!ev) return FA_ERR_NULL_POINTER;
    hipEvent_t e;
    FA_DEV(hipEventCreate(&e), "hipEventCreate");
    *ev = e;
    return FA_OK;
}
int fa_event_record(void *ev, void *stream) { FA_DEV(hipEventRecord(static_cast<hipEvent_t>(ev), static_cast<hipStream_t>(stream)), "hipEventRecord"); return FA_OK; }
int fa_event_sync(void *ev) { FA_DEV(hipEventSynchronize(static_cast<hipEvent_t>(ev)), "hipEventSynchronize"); return FA_OK; }
int fa_event_elapsed_ms(void *start, void *stop, float *ms)
{
    if (!ms) return FA_ERR_NULL_POINTER;
    FA_DEV(hipEventElapsedTime(ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)), "hipEventElapsedTime");
    return FA_OK;
}
int fa_event_destroy(void *ev) { FA_DEV(hipEventDestroy(static_cast<hipEvent_t>(ev)), "hipEventDestroy"); return FA_OK; }

// ---- backward pass (include/fa_bwd.h); the reference has none ----
unsigned long long fa_bwd_workspace_bytes(const fa_bwd_params *p)
{
    if (!p || p->B <= 0 || p->N <= 0 || p->S <= 0) return 0;
    return 2ull * (unsigned long long)p->B * p->N * p->S * 4ull;       // delta and the rescaled logsumexp
}

namespace {
// as many keys as queries, in any storage order and with any grouping of K/V heads; lengths that are a multiple of
// 128 also with dropout or with ALiBi (not both), other lengths without either
bool five_product_shape(const fa_bwd_params *p)
{
    if (p->S_kv != 0 && p->S_kv != p->S) return false;
    const bool alibi = p->alibi_slopes_ptr != nullptr, drop = fa_dropout_threshold(p->dropout_prob) != 0;
    return p->S % 128 == 0 ? !(alibi && drop) : !(alibi || drop);
}
unsigned long long ds_blocks_offset(const fa_bwd_params *p)
{
    return (fa_bwd_workspace_bytes(p) + 255ull) & ~255ull;
}
// K/V heads (counted through the batch) and the bytes of dS blocks that belong to one of them: those of its group
// of query heads
long long kv_heads_total(const fa_bwd_params *p) { return (long long)p->B * (p->n_kv_heads > 0 ? p->n_kv_heads : p->N); }
unsigned long long ds_bytes_per_kv_head(const fa_bwd_params *p)
{
    const int group = p->n_kv_heads > 0 ? p->N / p->n_kv_heads : 1;
    return (unsigned long long)group * (unsigned long long)fa_ds_blocks_per_head(p->S) * 2048ull;
}
// The fewest K/V heads a chunk of the five-product form may hold: enough key blocks for two rounds of a full chip,
// a multiple of eight (one head per XCD); all of them when the problem has no more.
long long min_chunk_kv_heads(const fa_bwd_params *p)
{
    const long long key_blocks = (p->S + 255) / 256, all = kv_heads_total(p);
    long long n = (2LL * kComputeUnits + key_blocks - 1) / key_blocks;
    n = (n + 7) / 8 * 8;
    return n < all ? n : all;
}
}  // namespace

unsigned long long fa_bwd_min_fast_workspace_bytes(const fa_bwd_params *p)
{
    if (fa_bwd_fast_workspace_bytes(p) == 0) return 0;
    return ds_blocks_offset(p) + (unsigned long long)min_chunk_kv_heads(p) * ds_bytes_per_kv_head(p);
}

unsigned long long fa_bwd_fast_workspace_bytes(const fa_bwd_params *p)
{
    if (!p || p->B <= 0 || p->N <= 0 || p->S <= 0 || (p->d != 64 && p->d != 128) || !five_product_shape(p)) return 0;
    return ds_blocks_offset(p) + (unsigned long long)p->B * p->N * (unsigned long long)fa_ds_blocks_per_head(p->S) * 2048ull;
}

int fa_bwd_validate(const fa_bwd_params *p)
{
    if (!p || !p->Q || !p->K || !p->V || !p->O || !p->dO || !p->L || !p->dQ || !p->dK || !p->dV) return FA_ERR_NULL_POINTER;
    if (p->B <= 0 || p->N <= 0 || p->S <= 0 || p->S_kv < 0) return FA_ERR_BAD_SHAPE;
    if (p->d != 64 && p->d != 128) return FA_ERR_HEAD_DIM;
    if (p->dtype != FA_DTYPE_F16 && p->dtype != FA_DTYPE_BF16) return FA_ERR_DTYPE;
    if (!(p->softmax_scale > 0.0f) || !isfinite(p->softmax_scale)) return FA_ERR_SCALE;
    if (p->n_kv_heads < 0 || (p->n_kv_heads > 0 && p->N % p->n_kv_heads != 0)) return FA_ERR_LAYOUT;
    if (!(p->dropout_prob >= 0.0f) || !(p->dropout_prob < 1.0f)) return FA_ERR_UNSUPPORTED;
    const long long s_kv = p->S_kv > 0 ? p->S_kv : p->S;
    if ((long long)p->B * p->N * ((p->S + 255) / 256) > 0x7fffffffLL || (long long)p->B * p->N * ((s_kv + 255) / 256) > 0x7fffffffLL ||
        (long long)p->S + s_kv > 0x3fffffffLL) return FA_ERR_TOO_LARGE;
    const void *ptrs[8] = {p->Q, p->K, p->V, p->O, p->dO, p->dQ, p->dK, p->dV};
    const long long *strides[8] = {p->q_strides, p->k_strides, p->v_strides, p->o_strides, p->do_strides,
                                   p->dq_strides, p->dk_strides, p->dv_strides};
    for (int t = 0; t < 8; ++t) {
        if (reinterpret_cast<uintptr_t>(ptrs[t]) % 16 != 0) return FA_ERR_LAYOUT;
        const long long *st = strides[t];
        if (st[0] == 0 && st[1] == 0 && st[2] == 0) continue;       // contiguous
        for (int k = 0; k < 3; ++k)
            if (st[k] < 0 || st[k] % 8 != 0) return FA_ERR_LAYOUT;
        if (st[2] < p->d) return FA_ERR_LAYOUT;
        if (st[2] > (1LL << 24)) return FA_ERR_TOO_LARGE;           // per-lane byte offsets inside a tile are 32-bit
        // a gradient whose batch or head stride is zero would have several writers per element
        if (t >= 5) {
            const int heads = t == 5 ? p->N : (p->n_kv_heads > 0 ? p->n_kv_heads : p->N);
            if ((p->B > 1 && st[0] == 0) || (heads > 1 && st[1] == 0)) return FA_ERR_LAYOUT;
        }
    }
    if (p->workspace == nullptr || reinterpret_cast<uintptr_t>(p->workspace) % 16 != 0 ||
        p->workspace_bytes < fa_bwd_workspace_bytes(p)) return FA_ERR_WORKSPACE;
    return FA_OK;
}

int fa_bwd(const fa_bwd_params *p, void *stream)
{
    const int st = fa_bwd_validate(p);
    if (st != FA_OK) return st;
    const FaDeviceState *ds = nullptr;
    {
        const hipError_t de = fa_device_state(&ds);
        if (de != hipSuccess) return device_fail(de, "device set-up");
    }
    FaBwdArgs a;
    a.Q = static_cast<const uint16_t *>(p->Q);
    a.K = static_cast<const uint16_t *>(p->K);
    a.V = static_cast<const uint16_t *>(p->V);
    a.O = static_cast<const uint16_t *>(p->O);
    a.dO = static_cast<const uint16_t *>(p->dO);
    a.lse = p->L;
    a.delta = static_cast<float *>(p->workspace);
    a.lse2 = a.delta + (size_t)p->B * p->N * p->S;
    // a workspace large enough for the dS blocks selects the five-product form
    // (all of them at once when it holds fa_bwd_fast_workspace_bytes, else for as many K/V heads' groups at a time as
    // fit, a multiple of eight and not fewer than fa_bwd_min_fast_workspace_bytes allows)
    const unsigned long long fast_bytes = fa_bwd_fast_workspace_bytes(p);
    a.ds_blocks = nullptr;
    a.head0 = 0;
    a.heads = (int)kv_heads_total(p);
    a.ds_heads = 0;
    if (fast_bytes != 0 && p->workspace_bytes >= fa_bwd_min_fast_workspace_bytes(p)) {
        const unsigned long long off = ds_blocks_offset(p);
        long long fit = (long long)((p->workspace_bytes - off) / ds_bytes_per_kv_head(p));
        if (fit < kv_heads_total(p)) fit = fit / 8 * 8;
        a.ds_heads = (int)(fit < kv_heads_total(p) ? fit : kv_heads_total(p));
        a.ds_blocks = reinterpret_cast<uint16_t *>(static_cast<char *>(p->workspace) + off);
    }
    a.dQ = static_cast<uint16_t *>(p->dQ);
    a.dK = static_cast<uint16_t *>(p->dK);
    a.dV = static_cast<uint16_t *>(p->dV);
    a.alibi = p->alibi_slopes_ptr;
    a.B = p->B;
    a.H = p->N;
    a.Hk = p->n_kv_heads > 0 ? p->n_kv_heads : p->N;
    a.S = p->S;
    a.Sk = p->S_kv > 0 ? p->S_kv : p->S;
    // general: any lengths, ALiBi, dropout; strided: the reference's lengths with other strides or grouped K/V heads
    // (drop_threshold is set further down: the same function of the probability)
    const bool general = a.S % 128 != 0 || a.Sk != a.S || (a.alibi != nullptr && fa_dropout_threshold(p->dropout_prob) != 0);
    bool strided = a.Hk != a.H;
    {
        const long long *strides[8] = {p->q_strides, p->k_strides, p->v_strides, p->o_strides, p->do_strides,
                                       p->dq_strides, p->dk_strides, p->dv_strides};
        FaBwdTensor *out[8] = {&a.q, &a.k, &a.v, &a.o, &a.dO_, &a.dq, &a.dk, &a.dv};
        for (int t = 0; t < 8; ++t) {
            const bool kv = t == 1 || t == 2 || t == 6 || t == 7;
            const long long heads = kv ? a.Hk : a.H, len = kv ? a.Sk : a.S;
            const long long dense[3] = {heads * len * p->d, len * p->d, p->d};
            const long long *st = strides[t];
            const bool given = st[0] != 0 || st[1] != 0 || st[2] != 0;
            long long eff[3];
            for (int k = 0; k < 3; ++k) {
                eff[k] = given ? st[k] : dense[k];
                if (eff[k] != dense[k]) strided = true;
            }
            out[t]->bs = eff[0]; out[t]->hs = eff[1]; out[t]->rs = (int)eff[2];
        }
    }
    // "unbounded" must stay unbounded after the shift by Sk - S that the key-owning kernel applies
    const int far = a.S + a.Sk;
    fa_mask_bounds(far, p->is_causal, p->window_size_left, p->window_size_right, &a.L, &a.R);
    a.scale = p->softmax_scale;
    a.drop_threshold = (unsigned)fa_dropout_threshold(p->dropout_prob);
    a.drop_scale = 256.0f / (256.0f - (float)a.drop_threshold);
    a.seed_lo = (unsigned)(p->seed & 0xffffffffull);
    a.seed_hi = (unsigned)(p->seed >> 32);
    const int masked = (general || a.L < far || a.R < far) ? 1 : 0;
    hipError_t e = (a.drop_threshold != 0 && !general)
        ? fa_launch_backward_dropout_regular(a, p->dtype == FA_DTYPE_BF16, p->d, masked, strided ? 1 : 0, ds->compute_units,
                                             static_cast<hipStream_t>(stream))
        : (a.alibi != nullptr && !general)
        ? fa_launch_backward_alibi_regular(a, p->dtype == FA_DTYPE_BF16, p->d, masked, strided ? 1 : 0, ds->compute_units,
                                           static_cast<hipStream_t>(stream))
        : a.drop_threshold != 0
        ? fa_launch_backward_dropout(a, p->dtype == FA_DTYPE_BF16, p->d, a.alibi != nullptr ? 1 : 0, ds->compute_units,
                                     static_cast<hipStream_t>(stream))
        : (strided && !general)
        ? fa_launch_backward_strided(a, p->dtype == FA_DTYPE_BF16, p->d, masked, ds->compute_units, static_cast<hipStream_t>(stream))
        : fa_launch_backward(a, p->dtype == FA_DTYPE_BF16, p->d, masked, general || strided ? 1 : 0, a.alibi != nullptr ? 1 : 0,
                             ds->compute_units, static_cast<hipStream_t>(stream));
    return e == hipSuccess ? FA_OK : device_fail(e, "backward launch");
}

void fa_bwd_sched_query_tile_range(int S, int S_kv, int is_causal, int window_left, int window_right,
                                   int k_begin, int rows, int *tile_lo, int *tile_hi)
{
    const int Sk = S_kv > 0 ? S_kv : S, off = Sk - S;
    int L, R;
    fa_mask_bounds(S + Sk, is_causal, window_left, window_right, &L, &R);
    fa_tile_range(S, 64, R + off, L - off, k_begin, rows, tile_lo, tile_hi);
}

int fa_bwd_sched_classify(int S, int S_kv, int is_causal, int window_left, int window_right,
                          int k_begin, int rows, int tile)
{
    const int Sk = S_kv > 0 ? S_kv : S, off = Sk - S;
    int L, R;
    fa_mask_bounds(S + Sk, is_causal, window_left, window_right, &L, &R);
    return fa_tile_class(64, R + off, L - off, k_begin, rows, tile);
}

// Five products over the unmasked pairs (the forward has two).  Square problems only, like fa_algorithmic_flops.
double fa_bwd_algorithmic_flops(int B, int N, int S, int d, int is_causal, int window_left, int window_right)
{
    return 2.5 * fa_algorithmic_flops(B, N, S, d, is_causal, window_left, window_right);
}

}  // extern "C"
