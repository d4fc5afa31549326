// Dropout on the regular problem (lengths a multiple of 128, as many keys as queries, no key splits): the strided
// instantiations' instruction stream -- three LDS stages, the next work item requested ahead, no ragged-edge code,
// strides and the K/V head of a work item from the arguments -- with DROPOUT = true, in a translation unit of its
// own.  Everything else with dropout takes the general instantiations (fa_fwd_kernel_dropout.hip).
#include "fa_fwd_kernel_impl.h"

hipError_t fa_launch_forward_dropout_regular(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                             hipStream_t stream)
{
    return launch_forward<false, true, true>(a, bf16, D, masked, shape, grid, stream);
}
hipError_t fa_configure_forward_dropout_regular() { return configure_forward<false, true, true>(); }
