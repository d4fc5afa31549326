// Instantiations of the forward kernel for the regular problem in a strided layout or with grouped K/V heads:
// lengths a multiple of 128, equal query and key lengths, no key splits, no dropout -- the reference's problem
// (reference src/flash_forward.h:593-665) with the tensors stored [B,S,N,d] or in any other layout with a
// contiguous head dimension, and with K/V heads that may be shared by groups of query heads.  The instruction
// stream is that of the contiguous instantiations (three LDS stages, the next work item requested ahead, no
// ragged-edge code) with batch, head and row strides taken from the arguments and the K/V head of a work item
// derived from its list position; the contiguous ones keep their compile-time addressing, which is worth 1-3 %
// to them.
#include "fa_fwd_kernel_impl.h"

hipError_t fa_launch_forward_strided(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                     hipStream_t stream)
{
    return launch_forward<false, false, true>(a, bf16, D, masked, shape, grid, stream);
}
hipError_t fa_configure_forward_strided() { return configure_forward<false, false, true>(); }
