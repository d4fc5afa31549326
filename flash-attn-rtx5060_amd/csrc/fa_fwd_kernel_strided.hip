// Instantiations of the forward kernel for the regular problem in a strided layout: lengths a multiple of 128,
// one K/V head per query head, equal query and key lengths, no key splits, no dropout -- the reference's problem
// (reference src/flash_forward.h:593-665) with the tensors stored [B,S,N,d] or in any other layout with a
// contiguous head dimension.  The instruction stream is that of the contiguous instantiations (three LDS stages,
// no ragged-edge or grouped-head code) with batch, head and row strides taken from the arguments; the
// contiguous ones keep their compile-time addressing, which is worth 1-3 % to them.
#include "fa_fwd_kernel_impl.h"

hipError_t fa_launch_forward_strided(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                     hipStream_t stream)
{
    return launch_forward<false, false, true>(a, bf16, D, masked, shape, grid, stream);
}
