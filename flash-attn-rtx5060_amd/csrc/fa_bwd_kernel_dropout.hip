// Backward kernels with dropout (general layout, with and without ALiBi), in a translation unit of their own.
#include "fa_bwd_kernel_impl.h"

hipError_t fa_launch_backward_dropout(const FaBwdArgs &a, int bf16, int D, int alibi, int compute_units, hipStream_t stream)
{
#define FA_BWD_CASE(BF, DD, AL) \
    if (bf16 == BF && D == DD && alibi == AL) return launch_bwd<BF != 0, DD, true, 2, AL != 0, true>(a, compute_units, stream);
    FA_BWD_CASE(0, 64, 0) FA_BWD_CASE(0, 128, 0) FA_BWD_CASE(1, 64, 0) FA_BWD_CASE(1, 128, 0)
    FA_BWD_CASE(0, 64, 1) FA_BWD_CASE(0, 128, 1) FA_BWD_CASE(1, 64, 1) FA_BWD_CASE(1, 128, 1)
#undef FA_BWD_CASE
    return hipErrorInvalidValue;
}
