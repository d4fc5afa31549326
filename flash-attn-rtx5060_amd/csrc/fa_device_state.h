// Per-device state of the library, set up once per device on the first call that needs it (or by fa_init):
// the device addresses of the library's two file-scope device arrays and the CU count.  Everything after that
// first call is a table lookup: no HIP query sits in the launch path.
#ifndef FA_DEVICE_STATE_H
#define FA_DEVICE_STATE_H
#include <hip/hip_runtime.h>

constexpr int kFaMaxDevices = 64;
constexpr int kFaEagerQueueSlots = 16;                         // counter sets for eager launches, one per stream
constexpr int kFaQueueSlots = 256;                             // work-queue counter sets per device; the rest serve captured launches
constexpr unsigned long long kFaStaticScratchBytes = 32ull << 20;   // key-split scratch per device

struct FaDeviceState {
    unsigned *queues;          // kFaQueueSlots sets of 16 words (nine used)
    unsigned char *scratch;    // kFaStaticScratchBytes bytes, 256-byte aligned
    int compute_units;
#ifdef FA_CHECK_RING
    unsigned long long *ring_check;     // checking build: comparisons made, mismatches found
#endif
};

// State of the current device (set up on first use).  Also records the device index for fa_launch_device().
hipError_t fa_device_state(const FaDeviceState **state);
// Index of the device the calling thread's current API call runs on (what fa_device_state saw last).
int fa_launch_device();

#endif
