/*
 * C ABI of the MI355X (gfx950) FlashAttention forward library, libfa_fwd_gfx950.so.
 *
 * Drop-in boundary for the reference operator `run_flash_attention`
 * (reference src/flash_forward.h:593-665) and its kernel argument block
 * `mykernelParamType` (reference include/utils.h:143-165).  Plain C types
 * only: device pointers are `void *`, booleans are `int`, the stream is an
 * opaque `void *` (a hipStream_t, NULL = the default stream).
 *
 * Tensors are contiguous [B, N, S, d] 16-bit (fp16 or bf16), exactly as the
 * reference lays them out (reference src/main.cu:182, flash_forward.h:378-381),
 * unless fa_fwd_params gives strides; the logsumexp output is fp32 [B, N, S].
 * d is 64 or 128; S is any positive length (the reference needs S % 128 == 0).
 */
#ifndef FA_FWD_H
#define FA_FWD_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* Status codes.  The reference exits, aborts, asserts or throws instead
 * (include/utils.h:16-23, flash_forward.h:384-387,587-589); nothing here
 * does: every entry point returns one of these. */
enum {
    FA_OK = 0,
    FA_ERR_NULL_POINTER = -1,      /* Q, K, V or O is NULL                                  */
    FA_ERR_BAD_SHAPE = -2,         /* B, N or S is not positive                              */
    FA_ERR_HEAD_DIM = -3,          /* d not in {64, 128}: reference throws, flash_forward.h:587 */
    FA_ERR_SEQLEN_MULTIPLE = -4,   /* reserved (was: S % 128 != 0, which the reference assumes silently,
                                      :134,637); any S >= 1 is accepted now                 */
    FA_ERR_UNSUPPORTED = -5,       /* dropout_prob is not in [0, 1)                          */
    FA_ERR_DTYPE = -6,             /* dtype is neither FA_DTYPE_F16 nor FA_DTYPE_BF16        */
    FA_ERR_SCALE = -7,             /* softmax_scale is not a finite positive number          */
    FA_ERR_DEVICE = -8,            /* a HIP runtime call failed; see fa_last_device_error()  */
    FA_ERR_NO_DEVICE = -9,         /* no gfx950 device is visible                            */
    FA_ERR_TOO_LARGE = -10,        /* B*N*S*d or the work-item count overflows the kernel's index range */
    FA_ERR_LAYOUT = -11,           /* a stride is not a multiple of 8 elements or too small, n_kv_heads does
                                      not divide N, or a tensor pointer is not 16-byte aligned */
    FA_ERR_WORKSPACE = -12,        /* split_num > 1 and the workspace is NULL, misaligned or too small */
    FA_ERR_SCRATCH_LIMIT = -13     /* fa_fwd_split_static: the partial results do not fit the static scratch */
};

enum { FA_DTYPE_F16 = 0, FA_DTYPE_BF16 = 1 };

/* How work items (batch, head, query block) reach the compute units. */
enum {
    FA_SCHED_AUTO = 0,        /* the library picks by the number of work items per resident
                                 workgroup: <= 1 dispatch, < 8 (or items all alike) persistent,
                                 else queue                                                    */
    FA_SCHED_DISPATCH = 1,    /* one workgroup per work item, launched longest-first          */
    FA_SCHED_PERSISTENT = 2,  /* a resident grid sized to the CUs walks the longest-first list
                                 in a fixed snake order                                       */
    FA_SCHED_QUEUE = 3        /* a resident grid takes items from the longest-first list
                                 through per-XCD counters in the library's own device memory  */
};

/*
 * Argument block.  The first twenty fields are those of the reference's
 * mykernelParamType (include/utils.h:143-165) in the same order with the same
 * meaning; the fields after `split_num` are what the reference passes as
 * template booleans (flash_forward.h:369) or hard-wires.
 */
typedef struct fa_fwd_params {
    const void *Q;            /* [B,N,S,d] device                                             */
    const void *K;
    const void *V;
    void *O;                  /* [B,N,S,d] device, fully overwritten                          */
    float *L;                 /* [B,N,S] fp32 logsumexp (natural log) or NULL.  The reference
                                 accepts L and never writes it (flash_forward.h:602,628-644). */
    float *M;                 /* unused, as in the reference; may be NULL                     */
    int B;
    int N;                    /* heads                                                        */
    int S;
    int d;
    int Tr;                   /* ignored on input (the reference derives them, :637-638)      */
    int Tc;
    float softmax_scale;      /* the reference sets 1/sqrt(d) itself, flash_forward.h:639     */
    float dropout_prob;       /* in [0, 1), applied in units of 1/256 (fa_dropout_threshold); 0 = none */
    unsigned long long seed;  /* dropout seed: the kept keys are a function of (seed, batch*N + head,
                                 query, key) alone, see fa_dropout_keep                       */
    void *states;             /* the reference's curand states (flash_forward.h:611): ignored */
    int window_size_left;     /* keys with i - j > left are masked;  < 0 = unbounded          */
    int window_size_right;    /* keys with j - i > right are masked; < 0 = unbounded          */
    const float *alibi_slopes_ptr; /* [N] device floats: score -= slope[h]*|i-j| (mask.h:21-26), or NULL */
    int split_num;            /* dead in the reference (utils.h:164).  Here: > 1 splits the keys of every
                                 (head, query block) into that many work items whose partial results a
                                 second kernel merges (long keys, few queries: decoding); needs
                                 `workspace`.  <= 1: one pass                                   */
    /* --- beyond mykernelParamType --- */
    int dtype;                /* FA_DTYPE_F16 / FA_DTYPE_BF16                                 */
    int is_causal;            /* keys with j > i are masked (mask.h:27-38)                    */
    int sched;                /* FA_SCHED_*                                                   */
    /* --- layouts beyond the reference's contiguous [B,N,S,d] (main.cu:182); all zero = that layout --- */
    int n_kv_heads;           /* K/V heads per batch entry, 0 = N.  Must divide N: query head h reads K/V
                                 head h / (N / n_kv_heads) (grouped-query / multi-query attention)      */
    long long q_strides[3];   /* batch, head and row (sequence position) strides of Q in elements; the
                                 head dimension is contiguous.  {0,0,0} = contiguous [B,N,S,d];
                                 a [B,S,N,d] tensor is {S*N*d, d, N*d}                                  */
    long long k_strides[3];   /* same for K ({0,0,0} = contiguous [B,n_kv_heads,S,d])                   */
    long long v_strides[3];
    long long o_strides[3];   /* same for O ({0,0,0} = contiguous [B,N,S,d]); L is always [B,N,S]       */
    int S_kv;                 /* keys per head when it differs from the S queries (0 = S).  K and V are
                                 [B, n_kv_heads, S_kv, d]; query i sits at key position i + S_kv - S (the
                                 queries are the last S positions), which is what the causal and window
                                 masks, the ALiBi distance and the dropout decision see.  Rows that see no
                                 key get O = 0 and L = -inf                                              */
    void *workspace;          /* device scratch for split_num > 1, at least fa_fwd_workspace_bytes()    */
    unsigned long long workspace_bytes;
    int exact_first_rows;     /* 0 (default): under a causal-type mask (no key right of the query) the query
                                 rows that see at most 32 keys are computed in the arithmetic of the
                                 reference's CPU verifier, every q*k and p*v product rounded to the storage
                                 type (main.cu:193,259): there an output can be as large as the values
                                 themselves and the verifier's own rounding, up to 3e-3 at unit variance, is
                                 larger than the tolerance a drop-in has to meet against it.  1: those rows
                                 use exact products and fp32 accumulation like every other row, and their
                                 logsumexp is the one a backward pass recomputes P from (fa_bwd)          */
} fa_fwd_params;

/* Checks a parameter block without touching any device.  Returns FA_OK or the
 * first violated FA_ERR_*.  (Replaces the reference's abort/throw/assert paths.) */
int fa_fwd_validate(const fa_fwd_params *p);

/* Device scratch a call with these parameters needs (0 unless split_num > 1):
 * splits * B * N * S * (d + 1) * 4 bytes of fp32 partial outputs and logsumexps. */
unsigned long long fa_fwd_workspace_bytes(const fa_fwd_params *p);
/* A split count that fills the device for these shapes (1 when the problem has enough work items anyway). */
int fa_fwd_suggest_splits(const fa_fwd_params *p);

/* Sets up the library's state for the current device: looks up the addresses of its two file-scope device
 * arrays and the CU count, and makes the LDS opt-in (hipFuncSetAttribute) of every kernel instantiation.  Optional
 * for eager use -- every entry point does what it still needs on its first call on a device -- but CALL IT BEFORE
 * A STREAM CAPTURE on that device: those first-call steps are not stream operations, and after fa_init() no
 * entry point makes any HIP call other than its kernel launches, hipStreamIsCapturing and hipStreamGetId. */
int fa_init(void);

/* Enqueues the forward pass on `stream` and returns without synchronising.
 * Allocates nothing; Q/K/V are read-only, O (and L when non-NULL) are
 * overwritten.  Re-entrant: the library keeps no per-call global state
 * (the reference keeps four global CUtensorMaps, flash_forward.h:17-20). */
int fa_fwd(const fa_fwd_params *p, void *stream);

/*
 * fa_fwd for callers that cannot allocate device memory.  No counterpart in the reference (which has no
 * key splits at all); it exists for callers under HIP graph capture, in tight serving loops or in harnesses
 * that forbid hipMalloc, who cannot provide the workspace a call with split_num > 1 needs.  Same arguments,
 * results and kernels as fa_fwd; `workspace` and `workspace_bytes` are ignored and the fp32 partial results
 * of the key splits go to a file-scope device array of fa_fwd_static_scratch_bytes() = 32 MiB that every
 * device holds for the life of the process.  Calls no allocating routine.  Returns FA_ERR_SCRATCH_LIMIT when
 * fa_fwd_workspace_bytes(p) exceeds that size.  All calls on one device share the array: two such calls that
 * overlap in time on one device (different streams, or a graph replay next to eager work) race; calls
 * ordered on one stream do not.  Nothing in the array has to start at zero: every partial row the merge
 * kernel reads is written by the launch before it.
 */
int fa_fwd_split_static(const fa_fwd_params *p, void *stream);
unsigned long long fa_fwd_static_scratch_bytes(void);

/* FA_SCHED_QUEUE keeps its counters in the library's own device memory: 256 sets per device; the last workgroup
 * of a launch rewinds its set.  Eager launches: a set belongs to a stream (launches on one stream run one after
 * the other and may share it), named by its handle and, where the loaded HIP runtime has hipStreamGetId (7.1 and
 * later), its runtime id, so that a new stream that happens to get a destroyed stream's handle value does not
 * inherit its set; with an older runtime the handle alone names it, and the release call below is required.  At most 16 streams of a device own
 * a set at a time; a stream keeps its set until fa_release_work_queue(stream) (call it before destroying a
 * stream that launched with the queue schedule; it waits for the stream) or fa_reset_work_queues().  Launches on
 * further streams, and on hipStreamPerThread (one handle value for a different stream in every host thread),
 * walk the work list with FA_SCHED_PERSISTENT's fixed order instead: same results, no counters.  Every launch
 * captured into a graph gets a set of its own, for good (a replay may run next to anything): 240 per device and
 * process, after which captured launches use the fixed order as well.  No two launches that can run at the same
 * time share counters.  A launch that was killed half-way (device reset, process signal) leaves its set dirty:
 * fa_reset_work_queues() waits for the device, zeroes all sets of the current device and forgets which stream
 * owned which.  Never call it while launches are being captured. */
int fa_reset_work_queues(void);
int fa_release_work_queue(void *stream);

/*
 * The reference's entry point, same name, argument order and meaning
 * (flash_forward.h:593-612; its only call site is src/main.cu:99):
 * fp16 tensors, softmax scale 1/sqrt(d), `Is_local` masks |i-j| > window_size
 * on both sides (mask.h:55-66), `Is_causal && Is_local` is "left window, right 0".
 * Like the reference it runs on the default stream of the current device and
 * returns after the kernel has finished (flash_forward.h:655); unlike it, it
 * prints nothing, returns a status, and fills L with the fp32 logsumexp when
 * L is non-NULL.  M is ignored.  `Has_alibi` takes `alibi_slopes` as N device floats and subtracts
 * slope[h]*|i-j| from every scaled score, once (mask.h:21-26; the reference applies it twice when causal
 * and local are both set).  `Is_dropout` applies dropout_prob with the fixed seed 48 (the seed main() gives its
 * curand states, main.cu:93); `states` is ignored: the kept keys come from a counter-based generator that a
 * host can replay (fa_dropout_keep), which curand states do not allow.
 */
int run_flash_attention(int B, int N, int S, int d,
                        void *Q, void *K, void *V, void *O,
                        void *L, void *M,
                        int Is_dropout, int Is_causal, int Is_local, int Has_alibi,
                        int window_size, float *alibi_slopes,
                        float dropout_prob, void *states);

/*
 * Dropout (reference flash_forward.h:248-265: after the softmax each probability is zeroed with probability p
 * or multiplied by 1/(1-p); the logsumexp is that of the undropped scores).  The decision for (bh = batch*N +
 * head, query i, key j) is byte 4*((j%32)/8) + j%4 of the Philox4x32-10 block with counter
 * (2*(j/32) + (j/4)%2, i, bh, 0x44524F50) and key (seed low, seed high): the key is kept iff that byte is >=
 * the threshold.  fa_dropout_threshold(p) = p rounded to 1/256 (at most 255); the factor applied to kept keys
 * is 256 / (256 - threshold).  Both are host functions: a backward pass or a test can replay the mask.
 */
int fa_dropout_threshold(float dropout_prob);
int fa_dropout_keep(unsigned long long seed, long long bh, int i, int j, int threshold);

const char *fa_strerror(int status);
/* Text of the last HIP error seen by the calling thread ("" if none). */
const char *fa_last_device_error(void);

/* ------------------------------------------------------------------ */
/* Tile scheduler, host side.  Mirrors what the kernel computes, so the */
/* schedule can be checked without a GPU.  Replaces Schedule<0,...>     */
/* (flash_forward.h:22-65).                                             */
/* ------------------------------------------------------------------ */
enum { FA_TILE_SKIP = 0, FA_TILE_PARTIAL = 1, FA_TILE_FULL = 2 };

/* Query rows per work item for a problem (128 or 256: it depends on how many keys a query can see, so the mask
 * is part of the question), and keys per tile for head dim d. */
int fa_sched_block_rows(int B, int N, int S, int d, int is_causal, int window_left, int window_right);
int fa_sched_block_keys(int d);
/* Number of work items for a problem: B*N*ceil(S/block_rows). */
long long fa_sched_num_items(int B, int N, int S, int d, int is_causal, int window_left, int window_right);
/* Work item `item` (0 = launched first) -> batch*N+head and first query row. */
int fa_sched_item(int B, int N, int S, int d, int is_causal, int window_left,
                  int window_right, long long item, int *bh, int *q_begin);
/* Grouped K/V heads of the regular problem (S a multiple of 128, S_kv = S, no key splits): the `bh` that
 * fa_sched_item returns is a position in the list of heads, and the kernel turns it into batch entry, query head
 * and K/V head like this (K/V heads fastest, so that the query heads of a K/V head share an XCD's L2).  With
 * n_kv_heads = 0 or N the position is the head.  No counterpart in the reference, which has one K/V head per
 * query head (flash_forward.h:378-381). */
int fa_sched_heads(int N, int n_kv_heads, int bh, int *batch, int *q_head, int *kv_head);
/* Key-tile range [*tile_lo, *tile_hi] (inclusive) visited for query rows
 * [q_begin, q_begin + rows).  Same clipping as flash_forward.h:52-61. */
void fa_sched_tile_range(int S, int block_keys, int is_causal, int window_left,
                         int window_right, int q_begin, int rows,
                         int *tile_lo, int *tile_hi);
/* Classification of key tile `tile` against query rows [q_begin, q_begin+rows). */
int fa_sched_classify(int block_keys, int is_causal, int window_left, int window_right,
                      int q_begin, int rows, int tile);
/* Unmasked (query, key) pairs per head, and algorithmic FLOPs 4*B*N*d*pairs. */
long long fa_count_pairs(int S, int is_causal, int window_left, int window_right);
double fa_algorithmic_flops(int B, int N, int S, int d, int is_causal,
                            int window_left, int window_right);

/* ------------------------------------------------------------------ */
/* Thin device layer so that a plain-C host harness needs no HIP header */
/* (the role cudaMalloc/cudaMemcpy/cudaEvent* play in src/main.cu:61-101 */
/* and flash_forward.h:646-662).                                        */
/* ------------------------------------------------------------------ */
int fa_dev_count(void);
int fa_dev_name(char *buf, size_t len, int *compute_units, int *clock_khz);
int fa_dev_malloc(void **ptr, size_t bytes);
int fa_dev_free(void *ptr);
int fa_dev_h2d(void *dst, const void *src, size_t bytes);
int fa_dev_d2h(void *dst, const void *src, size_t bytes);
int fa_dev_memset(void *dst, int value, size_t bytes);
int fa_dev_sync(void);
int fa_event_create(void **ev);
int fa_event_record(void *ev, void *stream);
int fa_event_sync(void *ev);
int fa_event_elapsed_ms(void *start, void *stop, float *ms);
int fa_event_destroy(void *ev);

#ifdef __cplusplus
}
#endif
#endif
