// The instantiations for everything else: strided tensors (for example [B,S,H,D]), query heads sharing K/V
// heads, sequence lengths that are not a multiple of 128.  Same kernel template, GENERAL = true.
#include "fa_fwd_kernel_impl.h"

hipError_t fa_launch_forward_general(const FaKernelArgs &a, int bf16, int D, int masked, int shape, unsigned grid,
                                     hipStream_t stream)
{
    return launch_forward<true, false>(a, bf16, D, masked, shape, grid, stream);
}
hipError_t fa_configure_forward_general() { return configure_forward<true, false>(); }

hipError_t fa_launch_combine_splits(const FaKernelArgs &a, int bf16, int D, hipStream_t stream)
{
    const long long n_rows = (long long)a.BH * a.S;
    const int rows_per_block = 256 / (D / 4);
    const unsigned grid = (unsigned)((n_rows + rows_per_block - 1) / rows_per_block);
    if (bf16 && D == 64) hipLaunchKernelGGL((fa_combine_splits<true, 64>), dim3(grid), dim3(256), 0, stream, a);
    else if (bf16) hipLaunchKernelGGL((fa_combine_splits<true, 128>), dim3(grid), dim3(256), 0, stream, a);
    else if (D == 64) hipLaunchKernelGGL((fa_combine_splits<false, 64>), dim3(grid), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((fa_combine_splits<false, 128>), dim3(grid), dim3(256), 0, stream, a);
    return hipGetLastError();
}
