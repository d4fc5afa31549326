// The instantiations for everything else: strided tensors (for example [B,S,H,D]), query heads sharing K/V
// heads, sequence lengths that are not a multiple of 128.  Same kernel template, GENERAL = true.
#include "fa_fwd_kernel_impl.h"

hipError_t fa_launch_forward_general(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                     hipStream_t stream)
{
    return launch_forward<true, false>(a, bf16, D, masked, shape, grid, stream);
}
