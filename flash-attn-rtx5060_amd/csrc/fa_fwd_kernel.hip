// The instantiations for contiguous [B,H,S,D] tensors with one K/V head per query head and S a multiple of
// 128 (the reference's only layout, src/main.cu:182), and the work-queue storage of the library.
#include "fa_fwd_kernel_impl.h"

// Work queues of FA_SCHED_QUEUE launches: kQueueSlots sets of nine counters, all zero between launches (the
// last workgroup of a launch rewinds its set).  Launches take the sets round-robin, so launches that overlap
// on one device do not share a set unless more than kQueueSlots of them are in flight at once.
constexpr int kQueueSlots = 32;
static __device__ __align__(256) unsigned g_work_queues[kQueueSlots][16];

hipError_t fa_work_queue_base(unsigned **base)
{
    return hipGetSymbolAddress(reinterpret_cast<void **>(base), HIP_SYMBOL(g_work_queues));
}
int fa_work_queue_slots() { return kQueueSlots; }

hipError_t fa_launch_forward_contiguous(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                        hipStream_t stream)
{
    return launch_forward<false, false>(a, bf16, D, masked, shape, grid, stream);
}
