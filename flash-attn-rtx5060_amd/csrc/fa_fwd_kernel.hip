// The instantiations for contiguous [B,H,S,D] tensors with one K/V head per query head and S a multiple of
// 128 (the reference's only layout, src/main.cu:182), and the work-queue storage of the library.
#include "fa_fwd_kernel_impl.h"

#include <atomic>
#include <mutex>

// Work queues of FA_SCHED_QUEUE launches: kFaQueueSlots sets of nine counters, all zero between launches (the
// last workgroup of a launch rewinds its set).  Which launch gets which set is the launcher's business
// (work_queue_for_launch in fa_fwd_api.hip): a set per stream for eager launches, a set of its own for every
// captured launch.
static __device__ __align__(256) unsigned g_work_queues[kFaQueueSlots][16];

// Scratch of fa_fwd_split_static: the fp32 partial outputs and logsumexps of a launch with key splits, for
// callers that may not allocate a workspace.  Every device holds its own copy for the life of the process.
// In host code the array's name is only a handle for hipGetSymbolAddress; kernels get the address it returns.
static __device__ __align__(256) unsigned char g_split_scratch[kFaStaticScratchBytes];

#ifdef FA_CHECK_RING
static __device__ __align__(16) unsigned long long g_ring_check[2];
#endif

namespace {
std::mutex g_state_mutex;
FaDeviceState g_state[kFaMaxDevices] = {};
std::atomic<bool> g_state_ready[kFaMaxDevices] = {};
thread_local int g_launch_device = 0;
}  // namespace

hipError_t fa_device_state(const FaDeviceState **state)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kFaMaxDevices) return hipErrorInvalidDevice;
    if (!g_state_ready[dev].load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(g_state_mutex);
        if (!g_state_ready[dev].load(std::memory_order_relaxed)) {
            // with `dev` current: each device holds its own copy of the arrays at its own address
            FaDeviceState st = {};
            e = hipGetSymbolAddress(reinterpret_cast<void **>(&st.queues), HIP_SYMBOL(g_work_queues));
            if (e != hipSuccess) return e;
            e = hipGetSymbolAddress(reinterpret_cast<void **>(&st.scratch), HIP_SYMBOL(g_split_scratch));
            if (e != hipSuccess) return e;
            if (st.queues == nullptr || st.scratch == nullptr) return hipErrorInvalidSymbol;
#ifdef FA_CHECK_RING
            e = hipGetSymbolAddress(reinterpret_cast<void **>(&st.ring_check), HIP_SYMBOL(g_ring_check));
            if (e != hipSuccess) return e;
#endif
            int n = 0;
            e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
            if (e != hipSuccess) return e;
            st.compute_units = n > 0 ? n : 256;
            g_state[dev] = st;
            g_state_ready[dev].store(true, std::memory_order_release);
        }
    }
    g_launch_device = dev;
    *state = &g_state[dev];
    return hipSuccess;
}
int fa_launch_device() { return g_launch_device; }

hipError_t fa_launch_forward_contiguous(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                        hipStream_t stream)
{
    return launch_forward<false, false>(a, bf16, D, masked, shape, grid, stream);
}
hipError_t fa_configure_forward_contiguous() { return configure_forward<false, false>(); }
