// The instantiations with dropout (reference src/flash_forward.h:248-265): the GENERAL kernel with DROPOUT = true.
#include "fa_fwd_kernel_impl.h"

hipError_t fa_launch_forward_dropout(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                     hipStream_t stream)
{
    return launch_forward<true, true>(a, bf16, D, masked, shape, grid, stream);
}
hipError_t fa_configure_forward_dropout() { return configure_forward<true, true>(); }
